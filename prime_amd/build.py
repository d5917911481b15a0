"""Compile libprime_hip.so for gfx950 with hipcc (cross-compiles without a GPU).

    python -m prime_amd.build

The library has no dependency besides the HIP runtime: no torch headers, no Python.
"""
from __future__ import annotations

import subprocess
import sys
from pathlib import Path

PKG = Path(__file__).resolve().parent
CSRC = PKG / "csrc"
LIB_PATH = CSRC / "libprime_hip.so"
SOURCES = [CSRC / "prime_hip.hip"]

HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-shared",
    "-ffp-contract=off",          # products and sums round separately unless fma() is written
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",   # no packed-fp32 instructions
    "-Wall",
]


def build(verbose: bool = True, defines: dict | None = None, out: Path | None = None) -> Path:
    """Compile the library.  ``defines`` overrides the PRIME_* tuning macros of the source and
    ``out`` redirects the output (for tuning sweeps that keep several variants side by side)."""
    out = Path(out) if out else LIB_PATH
    extra = [f"-D{k}={v}" for k, v in (defines or {}).items()]
    cmd = ["hipcc", *HIPCC_FLAGS, *extra, *map(str, SOURCES), "-o", str(out)]
    if verbose:
        print("+", " ".join(cmd), flush=True)
    subprocess.run(cmd, check=True)
    return out


if __name__ == "__main__":
    build()
    sys.exit(0)
