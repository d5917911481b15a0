"""Build recipe for the CPU oracle (test infrastructure, not product code).

    python oracle/build.py          # oracle/liboracle.so  (+ oracle/_ref when the reference is present)
    python oracle/build.py --no-ref

Two artefacts:

* ``oracle/liboracle.so``: the torch-free restatement in ``prime_oracle.cpp``, compiled
  with ``g++ -O3`` only, the single flag the reference builds its ops with
  (src/zeroband/C/compression.py:8).
* ``oracle/_ref/compression.so``: the reference's own ``src/zeroband/C/csrc/compression.cpp``
  compiled where it lies (nothing is copied) as the pybind11 module it declares
  (compression.cpp:129), against the libtorch of this image, the way
  ``torch.utils.cpp_extension.load`` would.  It validates the restatement and serves as the
  CPU baseline.  ``collectives.cpp`` is not built: it includes ProcessGroupGloo.hpp, whose
  gloo headers are an empty, un-vendored submodule of the reference.
"""
from __future__ import annotations

import argparse
import os
import subprocess
import sys
import sysconfig
from pathlib import Path

HERE = Path(__file__).resolve().parent
ORACLE_SO = HERE / "liboracle.so"
REF_DIR = HERE / "_ref"
REF_SO = REF_DIR / "compression.so"
REFERENCE_ROOT = Path(os.environ.get("PRIME_REFERENCE_ROOT", "/root/reference"))
REFERENCE_SRC = REFERENCE_ROOT / "src" / "zeroband" / "C" / "csrc" / "compression.cpp"


def _run(cmd: list[str]) -> None:
    print("+", " ".join(cmd), flush=True)
    subprocess.run(cmd, check=True)


def build_oracle() -> Path:
    _run(["g++", "-O3", "-std=c++17", "-shared", "-fPIC", "-pthread",
          str(HERE / "prime_oracle.cpp"), "-o", str(ORACLE_SO)])
    return ORACLE_SO


def build_ref() -> Path | None:
    """Compile the reference's compression.cpp in place; returns None when it is absent."""
    if not REFERENCE_SRC.exists():
        print(f"reference source {REFERENCE_SRC} not present: skipping oracle/_ref", flush=True)
        return None
    from torch.utils import cpp_extension  # include/library paths of the installed libtorch

    REF_DIR.mkdir(exist_ok=True)
    inc = [f"-I{p}" for p in cpp_extension.include_paths()]
    inc.append(f"-I{sysconfig.get_paths()['include']}")
    lib_dirs = cpp_extension.library_paths()
    cmd = ["g++", "-O3", "-std=c++17", "-shared", "-fPIC",
           "-DTORCH_API_INCLUDE_EXTENSION_H", "-DTORCH_EXTENSION_NAME=compression",
           *inc, str(REFERENCE_SRC), "-o", str(REF_SO)]
    for d in lib_dirs:
        cmd += [f"-L{d}", f"-Wl,-rpath,{d}"]
    cmd += ["-lc10", "-ltorch_cpu", "-ltorch", "-ltorch_python", "-pthread"]
    _run(cmd)
    return REF_SO


def main() -> None:
    ap = argparse.ArgumentParser()
    ap.add_argument("--no-ref", action="store_true")
    args = ap.parse_args()
    build_oracle()
    if not args.no_ref:
        build_ref()


if __name__ == "__main__":
    sys.exit(main())
