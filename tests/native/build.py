"""Build tests/native/abi_selftest: a host program (no Python, no torch) that calls the C ABI of
libprime_hip.so and checks it against the CPU oracle it is linked with.

    python tests/native/build.py
"""
from __future__ import annotations

import subprocess
import sys
from pathlib import Path

HERE = Path(__file__).resolve().parent
ROOT = HERE.parent.parent
BINARY = HERE / "abi_selftest"


def build(verbose: bool = True) -> Path:
    lib_dir = ROOT / "prime_amd" / "csrc"
    cmd = ["hipcc", "-O2", "-std=c++17", "-Wall", "-ffp-contract=off", f"-I{ROOT / 'include'}",
           str(HERE / "abi_selftest.cpp"), str(ROOT / "oracle" / "prime_oracle.cpp"),
           f"-L{lib_dir}", "-lprime_hip", "-Wl,-rpath,$ORIGIN/../../prime_amd/csrc", "-lpthread", "-o", str(BINARY)]
    if verbose:
        print("+", " ".join(cmd), flush=True)
    subprocess.run(cmd, check=True)
    return BINARY


if __name__ == "__main__":
    build()
    sys.exit(0)
