"""The ring all-reduce schedule on W simulated ranks (one GPU), through the host-side mirror
of the reference interface: ``all_reduce(Compression.UINT8, tensor, op, group)``."""
import math

import numpy as np
import pytest
import torch
import torch.distributed as dist

from tests.conftest import tables_agree
from tests.gpu_util import announce

pytestmark = pytest.mark.gpu

N = 1_000_000      # tests/test_c/test_collectives.py:13


def _inputs(W, n, seed):
    rng = np.random.default_rng(seed)
    return [(rng.standard_normal(n) * 10).astype(np.float32) for _ in range(W)]      # test_collectives.py:39


@pytest.mark.parametrize("W", [2, 4])
def test_ring_allreduce_matches_cpu_ring_like_the_reference_test(dev, oracle, W):
    # the reference's acceptance test (tests/test_c/test_collectives.py:14-57): the C ring and the
    # Python ring must land equally far from the exact all-reduce,
    # |norm(a - c) - norm(b - c)| / sqrt(N) < 0.5
    from prime_amd.C.collectives import SimulatedRing
    from prime_amd.collectives import Compression, all_reduce

    n = N - N % (2 * W)
    xs = _inputs(W, n, W)
    exact = np.sum(np.stack(xs).astype(np.float64), axis=0)
    cpu = [x.copy() for x in xs]
    oracle.ring_allreduce_sim(cpu, avg=False)
    announce(f"ring W={W}")
    gpu = [torch.from_numpy(x.copy()).to(dev) for x in xs]
    all_reduce(Compression.UINT8, gpu[0], dist.ReduceOp.SUM, SimulatedRing(gpu))
    torch.cuda.synchronize()
    for r in range(W):
        a = gpu[r].cpu().numpy()
        err_new = np.linalg.norm(a - exact)
        err_old = np.linalg.norm(cpu[r] - exact)
        assert abs(err_new - err_old) / math.sqrt(n) < 0.5
        # far tighter in fact: both are a fraction of one bin of the summed data
        assert abs(err_new - err_old) / math.sqrt(n) < 0.02
        assert err_new / math.sqrt(n) < 1.5 * (6 * 10 * math.sqrt(W) / 256) * math.sqrt(W - 1)


def test_ring_first_hop_is_bit_exact_against_cpu_ring(dev, oracle):
    # with W = 2 each chunk makes one hop; codes sent on step 1 are a pure function of the input
    from prime_amd import ring

    W, n = 2, 4 * 65536
    xs = _inputs(W, n, 9)
    gpu = [torch.from_numpy(x.copy()).to(dev) for x in xs]
    announce("ring first hop")
    csz = n // (2 * W)
    c = (0 * 2 - 1) % (2 * W)                       # rank 0, step 1 (collectives.cpp:116)
    chunk = gpu[0][c * csz:(c + 1) * csz]
    from tests.gpu_util import Abi

    abi = Abi(dev)
    codes, lut, qp = abi.uniform(chunk)
    q = abi.qparams(qp)
    oc, _, _ = oracle.uniform_8bit_quantize(xs[0][c * csz:(c + 1) * csz], "given", scale=float(q["scale"]))
    assert q["scale"] == oracle.scale_exact(xs[0][c * csz:(c + 1) * csz])
    assert np.array_equal(codes.cpu().numpy(), oc)
    ring.ring_allreduce_simulated(gpu)              # and the whole schedule runs


def test_ring_avg_and_single_rank(dev, oracle):
    from prime_amd.C.collectives import SimulatedRing, ring_allreduce

    W, n = 4, 8 * 4096
    xs = _inputs(W, n, 3)
    gpu = [torch.from_numpy(x.copy()).to(dev) for x in xs]
    announce("ring AVG")
    ring_allreduce(gpu[1], dist.ReduceOp.AVG, SimulatedRing(gpu))
    exact = np.mean(np.stack(xs).astype(np.float64), axis=0)
    for t in gpu:
        assert np.linalg.norm(t.cpu().numpy() - exact) / math.sqrt(n) < 6 * 10 / 256
    # one rank: no message, but the rank's two chunks take the quantize / dequantize round trip
    x = xs[0]
    t = torch.from_numpy(x.copy()).to(dev)
    announce("ring W=1")
    ring_allreduce(t, dist.ReduceOp.SUM, SimulatedRing([t]))
    want = [x.copy()]
    oracle.ring_allreduce_sim(want)
    got = t.cpu().numpy()
    assert len(np.unique(got[: n // 2])) <= 256 and len(np.unique(got[n // 2:])) <= 256
    assert np.allclose(got, want[0], rtol=2e-6, atol=1e-6)
    codes_a = oracle.uniform_8bit_quantize(x[: n // 2], "exact")[0]
    # dequantized values map one-to-one onto the oracle's codes
    assert len(np.unique(codes_a)) == len(np.unique(got[: n // 2]))


@pytest.mark.parametrize("W,avg", [(2, True), (3, True), (4, False), (8, True)])
def test_whole_schedule_tracks_the_cpu_ring_element_by_element(dev, oracle, W, avg):
    # Same schedule, same arithmetic: the two runs differ only through lookup entries that
    # agree to 1e-6, which moves a value across a bin edge now and then.  Nearly every element
    # must agree to float rounding, and none may be further than a bin or two away.
    from prime_amd import ring

    n = 2 * W * 20_000
    xs = _inputs(W, n, 100 + W)
    cpu = [x.copy() for x in xs]
    oracle.ring_allreduce_sim(cpu, avg=avg)
    announce(f"ring element-wise W={W} avg={avg}")
    gpu = [torch.from_numpy(x.copy()).to(dev) for x in xs]
    ring.ring_allreduce_simulated(gpu, avg=avg)
    torch.cuda.synchronize()
    bin_width = 6 * 10 * math.sqrt(W) / 256 / (W if avg else 1)
    for r in range(W):
        d = np.abs(gpu[r].cpu().numpy() - cpu[r])
        assert d.max() < 2.5 * bin_width
        assert (d > 1e-2 * bin_width).mean() < 2e-3
    # every rank ends with the same tensor except for the chunks it did not requantize last
    ref_t = gpu[0].cpu().numpy()
    for r in range(1, W):
        assert np.abs(gpu[r].cpu().numpy() - ref_t).max() < 2.5 * bin_width


@pytest.mark.parametrize("W,avg,n", [(2, False, 100_003), (3, True, 100_001), (4, False, 1_000_001), (8, True, 262_147), (4, True, 29)])
def test_a_tensor_that_2w_does_not_divide_is_cut_as_torch_chunk_cuts_it(dev, oracle, W, avg, n):
    # collectives.cpp:89-90 cuts with flat.chunk(2 W): pieces of ceil(n / 2W), the last one shorter.  The whole
    # schedule on such a tensor against the oracle ring (same cut), element by element as above, through the
    # lock-stepped ring, the staged ring (messages of two sizes through the pinned slots) and with the
    # closed form: inputs constant on every chunk come back as the exact sums
    from prime_amd import ring, wire
    from prime_amd.ring import chunk_bounds

    bounds = chunk_bounds(n, W)
    assert len(bounds) == 2 * W and bounds[-1][1] == n and bounds[-1][1] - bounds[-1][0] < bounds[0][1] - bounds[0][0]
    assert bounds == oracle.torch_chunk_bounds(n, 2 * W)
    assert [b - a for a, b in bounds] == [c.numel() for c in torch.empty(n).chunk(2 * W)]
    xs = _inputs(W, n, 300 + W)
    cpu = [x.copy() for x in xs]
    oracle.ring_allreduce_sim(cpu, avg=avg)
    announce(f"ring with a shorter last chunk W={W} avg={avg} n={n}")
    gpu = [torch.from_numpy(x.copy()).to(dev) for x in xs]
    ring.ring_allreduce_simulated(gpu, avg=avg)
    staged = [torch.from_numpy(x.copy()).to(dev) for x in xs]
    wire.ring_allreduce_staged(staged, avg=avg)
    torch.cuda.synchronize()
    bin_width = 6 * 10 * math.sqrt(W) / 256 / (W if avg else 1)
    for r in range(W):
        assert torch.equal(staged[r], gpu[r])
        d = np.abs(gpu[r].cpu().numpy() - cpu[r])
        assert d.max() < 2.5 * bin_width
        if n > 1000:
            assert (d > 1e-2 * bin_width).mean() < 2e-3
    # closed form: rank r holds v[r, c] on chunk c; a constant quantizes without loss, so every rank ends with the
    # exact sum over the ranks on every chunk (a wrong boundary would mix two constants)
    if bounds[-1][1] - bounds[-1][0] > 1:
        vals = np.arange(1, W * 2 * W + 1, dtype=np.float32).reshape(W, 2 * W)
        flat = []
        for r in range(W):
            t = np.empty(n, np.float32)
            for c, (a, b) in enumerate(bounds):
                t[a:b] = vals[r, c]
            flat.append(torch.from_numpy(t).to(dev))
        ring.ring_allreduce_simulated(flat, avg=False)
        want = np.empty(n, np.float32)
        for c, (a, b) in enumerate(bounds):
            want[a:b] = vals[:, c].sum()
        for r in range(W):
            assert np.array_equal(flat[r].cpu().numpy(), want), r
    with pytest.raises(ValueError, match="split into"):
        ring.ring_allreduce_simulated([torch.zeros(2 * W + 1, device=dev) for _ in range(W)] if W > 1 else [torch.zeros(1, device=dev)])


@pytest.mark.parametrize("W,avg", [(1, False), (2, True), (4, False), (8, True)])
def test_all_gather_in_the_code_domain_gives_the_same_tensors(dev, W, avg):
    # keep_codes: what is forwarded is requantized from the received codes alone and the fp32 chunk is
    # never written; a rank's result is lut[codes] of what it received.  Codes are identical to the
    # plain schedule's; lookup entries agree to rounding, which can move an element across a bin edge
    from prime_amd import ops, ring

    n = 2 * W * 30_000
    xs = _inputs(W, n, 200 + W)
    plain = [torch.from_numpy(x.copy()).to(dev) for x in xs]
    coded = [torch.from_numpy(x.copy()).to(dev) for x in xs]
    announce(f"ring keep_codes W={W} avg={avg}")
    ring.ring_allreduce_simulated(plain, avg=avg)
    final = ring.ring_allreduce_simulated(coded, avg=avg, keep_codes=True)
    torch.cuda.synchronize()
    assert len(final) == W and all(len(f) == 2 * W for f in final)
    bin_width = 6 * 10 * math.sqrt(W) / 256 / (W if avg else 1)
    for r in range(W):
        got = torch.cat([ops.dequantize(c, l) for c, l in final[r]])
        d = (got - plain[r]).abs().cpu().numpy()
        assert d.max() < 2.5 * bin_width
        assert (d > 1e-2 * bin_width).mean() < 2e-3
        for c, l in final[r]:
            assert c.dtype == torch.uint8 and c.numel() == n // (2 * W) and l.shape == (256,)
    # a rank's own chunks never travelled: bit-identical
    csz = n // (2 * W)
    for r in range(W):
        for i in range(2):
            c = 2 * r + i
            assert torch.equal(ops.dequantize(*final[r][c]), plain[r][c * csz:(c + 1) * csz])


def test_ops_layer_checks_on_device_tensors(dev):
    from prime_amd.C import compression as C
    from prime_amd import ops

    x = torch.randn(1000, device=dev)
    with pytest.raises(RuntimeError, match="Float"):
        C.uniform_8bit_quantize(x.double())
    with pytest.raises(RuntimeError, match="Byte"):
        C.average_buckets(x, torch.zeros(1000, dtype=torch.int32, device=dev), 256)
    with pytest.raises(RuntimeError, match="numel"):
        C.average_buckets(x, torch.zeros(10, dtype=torch.uint8, device=dev), 256)
    codes, lut = C.uniform_8bit_quantize(x.view(10, 100))
    assert codes.shape == (10, 100) and codes.dtype == torch.uint8 and lut.shape == (256,)
    # a non-contiguous input is read in logical order, never modified
    xt = torch.randn(64, 32, device=dev)
    before = xt.clone()
    c1, l1 = C.uniform_8bit_quantize(xt.t(), True)
    c2, l2 = C.uniform_8bit_quantize(xt.t().contiguous(), True)
    assert torch.equal(c1, c2) and torch.equal(l1, l2) and torch.equal(xt, before)
    with pytest.raises(RuntimeError, match="contiguous"):
        ops.dequantize_(torch.zeros(64, 32, device=dev).t(), c1, l1, False)
    q = C.quantize_per_tensor_uint8(torch.ones(1000, device=dev) * 10, 0.01, 128)
    assert bool((q == 255).all())
    d = ops.dequantize(c1, l1)
    assert torch.equal(d, l1[c1.long()])


def test_norm_mode_switch_of_the_compression_module(dev, oracle):
    # set_norm_mode("libtorch"): uniform_8bit_quantize gives the scale-dependent codes of a CPU run of the
    # reference (oracle in literal mode, itself pinned against torch's norm and the compiled reference)
    from prime_amd.C import compression as C

    rng = np.random.default_rng(12)
    x = (rng.standard_normal(3_000_003) * 1e-3).astype(np.float32)
    t = torch.from_numpy(x).to(dev)
    assert C.get_norm_mode() == "exact"
    announce("norm mode switch")
    try:
        C.set_norm_mode("libtorch")
        c_lit, _ = C.uniform_8bit_quantize(t)
    finally:
        C.set_norm_mode("exact")
    c_exact, _ = C.uniform_8bit_quantize(t)
    assert np.array_equal(c_lit.cpu().numpy(), oracle.uniform_8bit_quantize(x, "literal")[0])
    assert np.array_equal(c_exact.cpu().numpy(), oracle.uniform_8bit_quantize(x, "exact")[0])
    assert not torch.equal(c_lit, c_exact)          # libtorch's norm is off by 1e-4 here: a few codes move
    with pytest.raises(ValueError):
        C.set_norm_mode("fast")


def test_div_kernel_is_fp32_division(dev, oracle):
    # chunk.div_(world_size) of ReduceOp::AVG (collectives.cpp:155-159)
    from prime_amd import ops

    rng = np.random.default_rng(19)
    for n in (1, 6, 4097, 1_000_001):
        x = rng.standard_normal(n).astype(np.float32)
        for d in (2.0, 3.0, 14.0):
            t = torch.from_numpy(x.copy()).to(dev)
            ops.div_(t, d)
            want = x.copy()
            oracle.div_scalar(want, d)
            assert np.array_equal(t.cpu().numpy(), want)


def test_reference_import_paths_reach_the_hip_kernels(dev):
    # the body of the reference's own tests/test_c/test_compression.py (:14-56), with its imports
    # unchanged, after prime_amd.shim.install()
    import sys

    import prime_amd.shim as shim

    shim.install()
    try:
        from zeroband.C.compression import average_buckets, quantize_per_tensor_uint8, uniform_8bit_quantize

        N = 1_000_000
        announce("reference import paths")
        a = torch.randn(N, device=dev) * 10
        codes, lut = uniform_8bit_quantize(a)
        assert codes.dtype == torch.uint8 and codes.shape == a.shape and lut.shape == (256,)
        diff = (lut[codes.long()] - a).abs()
        assert float(diff.max()) <= 6 * float(a.norm() / math.sqrt(N - 1)) / 256 * 1.01 or float(diff.median()) < 0.2
        # the table of the fused pass (fixed-point residual sums) and that of average_buckets (fp64 sums)
        # are both within 1e-6 of the exact bin means
        new_lut = average_buckets(a, codes, 256)
        scale = 6 * float(a.norm() / math.sqrt(N - 1)) / 256
        assert tables_agree(new_lut.cpu().numpy(), lut.cpu().numpy(), scale, 2e-6)
        q = quantize_per_tensor_uint8(torch.ones(N, device=dev) * 10, 0.01, 128)
        assert bool((q == 255).all())
    finally:
        shim.uninstall()
        for k in [k for k in sys.modules if k == "zeroband" or k.startswith("zeroband.")]:
            del sys.modules[k]


@pytest.mark.parametrize("W", [1, 2, 3, 4, 5, 7, 8])
@pytest.mark.parametrize("avg", [False, True])
@pytest.mark.parametrize("code_domain", [False, True])
def test_ring_closed_form_on_chunkwise_constant_inputs(dev, W, avg, code_domain):
    # rank r's chunk c is a constant; constant chunks quantize without loss and every partial sum is a
    # small integer, so the ring must return exactly sum_r v[r, c] (divided by W for AVG) in every
    # element of chunk c on every rank: pins the chunk-index algebra (collectives.cpp:116, 192), the
    # forwarding condition (:136, :212), the division (:155-159) and the own-chunk round trip
    # (:161-173) bit for bit, with the same inputs as the oracle's own closed-form test
    from prime_amd import ops, ring
    from tests.test_oracle_pins import closed_form_ring_inputs

    csz = 4096
    v, tensors = closed_form_ring_inputs(W, csz)
    announce(f"closed-form ring W={W} avg={avg} code_domain={code_domain}")
    gpu = [torch.from_numpy(t).to(dev) for t in tensors]
    final = ring.ring_allreduce_simulated(gpu, avg=avg, keep_codes=code_domain)
    torch.cuda.synchronize()
    total = v.sum(axis=0, dtype=np.float64).astype(np.float32)
    want = total / np.float32(W) if avg else total
    for rk in range(W):
        if code_domain:
            got = np.stack([ops.dequantize(*final[rk][c]).cpu().numpy() for c in range(2 * W)])
        else:
            got = gpu[rk].cpu().numpy().reshape(2 * W, csz)
        for c in range(2 * W):
            assert np.all(got[c] == want[c]), (W, avg, rk, c, got[c][:3], want[c])


@pytest.mark.parametrize("n", [3, 7, 1001, 65537])
def test_single_rank_group_takes_an_odd_number_of_elements(dev, oracle, n):
    # flat.chunk(2) of the reference's C++ (collectives.cpp:90): ceil(n / 2) elements and the rest, each
    # through the quantize / dequantize round trip (:161-173)
    from prime_amd import ring

    rng = np.random.default_rng(n)
    x = (rng.standard_normal(n) * 1e-3).astype(np.float32)
    t = torch.from_numpy(x.copy()).to(dev)
    announce(f"single rank odd n={n}")
    ring.ring_allreduce_single(t)
    torch.cuda.synchronize()
    (lo0, hi0), (lo1, hi1) = oracle.torch_chunk_bounds(n, 2)
    want = x.copy()
    for lo, hi in ((lo0, hi0), (lo1, hi1)):
        codes, _, scale = oracle.uniform_8bit_quantize(x[lo:hi], "exact")
        mean, _ = oracle.average_buckets_f64(x[lo:hi], codes)
        want[lo:hi] = mean.astype(np.float32)[codes]
    got = t.cpu().numpy()
    floor = 6 * 1e-3 / 256
    assert np.all(np.abs(got - want) <= 1e-6 * np.maximum(np.abs(want), floor))
    with pytest.raises(ValueError):
        ring.ring_allreduce_single(torch.zeros(1, device=dev))
