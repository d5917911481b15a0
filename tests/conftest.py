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
    bins whose mean is near zero (the centre bin straddles zero)."""
    lut = np.asarray(lut, np.float64)
    denom = np.maximum(np.abs(mean64), float(scale))
    with np.errstate(invalid="ignore"):
        e = np.abs(lut - mean64) / denom
    return float(np.nanmax(e)) if e.size else 0.0
