import sys
from pathlib import Path

import numpy as np
import pytest

ROOT = Path(__file__).resolve().parents[1]
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def oracle():
    """The CPU oracle; built on demand where only the source travelled."""
    from oracle import oracle as O

    if not O._LIB_PATH.exists():
        from oracle import build as ob

        ob.build_oracle()
    return O


@pytest.fixture(scope="session")
def golden():
    return np.load(ROOT / "tests" / "golden" / "uniform8_reference.npz")


@pytest.fixture(scope="session")
def dev():
    import torch

    assert torch.cuda.is_available(), "GPU tests need a ROCm device"
    return torch.device("cuda:0")


def lut_rel_err(lut, mean64, scale):
    """max |lut - mean| / max(|mean|, scale): 1e-6 relative, with the bin width as the floor for
    bins whose mean is near zero (the centre bin straddles zero).  An entry that is not a number
    where the mean is one (or the reverse), or a different infinity, counts as an infinite error."""
    lut = np.asarray(lut, np.float64)
    mean64 = np.asarray(mean64, np.float64)
    if lut.shape != mean64.shape:
        return float("inf")
    if not lut.size:
        return 0.0
    if not np.array_equal(np.isnan(lut), np.isnan(mean64)):
        return float("inf")
    special = ~np.isfinite(mean64) | ~np.isfinite(lut)
    sp_ok = np.array_equal(lut[special & ~np.isnan(mean64)], mean64[special & ~np.isnan(mean64)])
    if not sp_ok:
        return float("inf")
    fin = ~special
    if not fin.any():
        return 0.0
    denom = np.maximum(np.abs(mean64[fin]), float(scale))
    return float(np.max(np.abs(lut[fin] - mean64[fin]) / denom))


def tables_agree(a, b, scale, tol):
    """Two lookup tables that are each within the bar of the same fp64 means: |a - b| <= tol *
    max(|b|, one bin width), entry by entry, with the same NaN and infinite entries."""
    floor = float(scale) if np.isfinite(scale) and scale > 0 else 1.0
    return lut_rel_err(np.asarray(a, np.float64), np.asarray(b, np.float64), floor) <= tol
