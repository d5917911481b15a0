"""The one configuration value the compression path reads.

Mirrors ``Compression`` in the reference (src/zeroband/config.py:10-12): the value
strings are what its TOML files and ``ZERO_BAND_DILOCO_COMPRESSION`` carry.
"""
from enum import Enum


class Compression(Enum):
    NO = "no"
    UINT8 = "uint8"
