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


def kernel_resources() -> dict:
    """Registers and scratch of every kernel as the production flags compile it: a device-only
    compile with the compiler's resource remarks.  Returns {mangled name: {"vgprs", "scratch",
    "occupancy", "lds"}}.  A streaming kernel that needs scratch has spilled registers: its spill
    traffic competes with the data it streams."""
    import re
    import tempfile

    flags = [f for f in HIPCC_FLAGS if f not in ("-shared", "-fPIC")]
    with tempfile.TemporaryDirectory() as tmp:
        cmd = ["hipcc", *flags, "--cuda-device-only", "-c", *map(str, SOURCES), "-o", str(Path(tmp) / "device.o"),
               "-Rpass-analysis=kernel-resource-usage"]
        res = subprocess.run(cmd, check=True, capture_output=True, text=True)
    out, name = {}, None
    keys = {"VGPRs": "vgprs", "ScratchSize [bytes/lane]": "scratch", "Occupancy [waves/SIMD]": "occupancy",
            "LDS Size [bytes/block]": "lds"}
    for line in res.stderr.splitlines():
        m = re.search(r"Function Name: (\S+)", line)
        if m:
            name = m.group(1)
            out[name] = {}
            continue
        for label, key in keys.items():
            m = re.search(re.escape(label) + r": (\d+)", line)
            if m and name:
                out[name][key] = int(m.group(1))
    return out


def device_data_symbols() -> dict:
    """Data objects of the gfx950 code object as the production flags compile it:
    {symbol name: {"size", "bind"}}.  A __device__ variable that host code looks up by symbol
    (hipGetSymbolAddress) must be GLOBAL there: the runtime resolves it through the code object's
    dynamic symbols and aborts the process when the name is missing."""
    import tempfile

    flags = [f for f in HIPCC_FLAGS if f not in ("-shared", "-fPIC")]
    llvm = Path("/opt/rocm/llvm/bin")
    with tempfile.TemporaryDirectory() as tmp:
        obj, co = Path(tmp) / "device.o", Path(tmp) / "device.co"
        subprocess.run(["hipcc", *flags, "--cuda-device-only", "-c", *map(str, SOURCES), "-o", str(obj)],
                       check=True, capture_output=True)
        subprocess.run([str(llvm / "clang-offload-bundler"), "--unbundle", "--type=o", f"--input={obj}",
                        "--targets=hip-amdgcn-amd-amdhsa--gfx950", f"--output={co}"], check=True, capture_output=True)
        res = subprocess.run([str(llvm / "llvm-readelf"), "--dyn-syms", str(co)], check=True, capture_output=True, text=True)
    out = {}
    for line in res.stdout.splitlines():
        f = line.split()
        if len(f) == 8 and f[3] == "OBJECT" and not f[7].endswith(".kd"):
            out[f[7]] = {"size": int(f[2]), "bind": f[4]}
    return out


if __name__ == "__main__":
    build()
    sys.exit(0)
