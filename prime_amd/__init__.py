"""prime_amd: the int8 pseudo-gradient compression path of prime (ZeroBand) on MI355X.

Layout
    csrc/            HIP kernels (kernels_*.h, device_common.h) and the C ABI (prime_hip.hip ->
                     libprime_hip.so; include/prime_hip.h)
    _lib.py          ctypes binding of the C ABI
    ops.py           torch.library ops over it
    C/compression.py, C/collectives.py, collectives.py, config.py
                     the reference's module and function names for this path
    ring.py          the ring's per-hop compute for W simulated ranks on one GPU
    diloco.py        pseudo-gradient, bucketing and outer step around the all-reduce, GPU-resident
    wire.py          message layout and pinned host staging between the GPU and a host transport
    shim.py          registers these modules under the reference's import paths (zeroband.*)
"""
from .config import Compression  # noqa: F401

__all__ = ["Compression"]
