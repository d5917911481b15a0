"""The entry point that allocates nothing (prime_uniform_8bit_quantize_noalloc) against
prime_uniform_8bit_quantize with a caller's workspace, through the C ABI: codes, lookup table
and statistics record bit for bit, on two calls in a row, the second on a smaller input (the
built-in scratch keeps the first call's partials)."""
import numpy as np
import pytest
import torch

from prime_amd import _lib
from tests.gpu_util import Abi, announce

pytestmark = pytest.mark.gpu


def _noalloc(abi, x):
    n = x.numel()
    codes = torch.empty(n, dtype=torch.uint8, device=abi.dev)
    lut = torch.empty(256, dtype=torch.float32, device=abi.dev)
    qp = torch.empty(4, dtype=torch.float64, device=abi.dev)
    _lib.check(abi.lib.prime_uniform_8bit_quantize_noalloc(x.data_ptr(), n, codes.data_ptr(), lut.data_ptr(), qp.data_ptr(),
                                                           abi.st), "uniform_noalloc")
    return codes, lut, qp


def test_noalloc_entry_point_equals_the_workspace_one_twice_in_a_row(dev):
    abi = Abi(dev)
    rng = np.random.default_rng(77)
    sizes = ((1 << 22) + 5, 70_001)            # 513 workgroups' worth of partials, then 18
    xs = [abi.to_dev((rng.standard_normal(n) * 1e-3).astype(np.float32)) for n in sizes]
    for n, x in zip(sizes, xs):
        announce(f"noalloc n={n}")
        gc, gl, gq = _noalloc(abi, x)
        torch.cuda.synchronize()
        wc, wl, wq = abi.uniform(x)
        torch.cuda.synchronize()
        assert torch.equal(gc, wc), n
        # the histogram partials are integer sums (no element here lies beyond the fixed-point range), so the
        # table does not depend on the order of the LDS additions: bit for bit, as the header promises
        assert np.array_equal(gl.cpu().numpy().view(np.uint32), wl.cpu().numpy().view(np.uint32)), n
        assert np.array_equal(gq.cpu().numpy().view(np.uint64), wq.cpu().numpy().view(np.uint64)), n
        assert abi.qparams(gq)["n"] == n


def test_noalloc_rejects_what_it_cannot_hold(dev):
    abi = Abi(dev)
    lut = torch.empty(256, dtype=torch.float32, device=dev)
    rc = abi.lib.prime_uniform_8bit_quantize_noalloc(lut.data_ptr(), (1 << 40) + 1, lut.data_ptr(), lut.data_ptr(), None, abi.st)
    assert rc == -1 and b"2^40" in abi.lib.prime_hip_last_error()
    assert abi.lib.prime_uniform_8bit_quantize_noalloc(None, 16, None, lut.data_ptr(), None, abi.st) == -1
