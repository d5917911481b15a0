"""The C ABI used from a plain C++ host program: no Python, no torch in the process that calls
the library (tests/native/abi_selftest.cpp, built by tests/native/build.py)."""
import subprocess
from pathlib import Path

import pytest

from tests.gpu_util import announce

pytestmark = pytest.mark.gpu

BINARY = Path(__file__).resolve().parent / "native" / "abi_selftest"


def test_native_host_program_passes_its_checks(dev):
    assert BINARY.exists(), f"{BINARY} is not built: run `python tests/native/build.py` (or __graft_entry__.build())"
    announce("native C-ABI self-test")
    res = subprocess.run([str(BINARY)], capture_output=True, text=True, timeout=120)
    print(res.stdout)
    print(res.stderr)
    assert res.returncode == 0, res.stdout[-2000:] + res.stderr[-2000:]
    assert "all checks passed" in res.stdout and "FAILED" not in res.stdout
