"""The callers either side of the compression path: pseudo-gradient, outer optimizer step and
the GPU-resident Diloco state (src/zeroband/diloco.py), against the oracle and against torch's
own CPU SGD."""
import math

import numpy as np
import pytest
import torch
from torch import nn

from tests.gpu_util import announce

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("n", [1, 5, 1023, 4096, 1_000_003])
def test_pseudo_gradient_kernel_bit_exact(dev, oracle, n):
    from prime_amd import ops

    rng = np.random.default_rng(n)
    a = rng.standard_normal(n).astype(np.float32)
    b = (a + rng.standard_normal(n).astype(np.float32) * 1e-3).astype(np.float32)
    announce(f"pseudo gradient n={n}")
    for W in (1.0, 3.0, 8.0):
        out = torch.empty(n, device=dev)
        ops.pseudo_gradient_(out, torch.from_numpy(a).to(dev), torch.from_numpy(b).to(dev), W)
        assert np.array_equal(out.cpu().numpy(), oracle.pseudo_gradient(a, b, W))
    # misaligned views take the element-aligned kernel
    big = torch.zeros(3 * (n + 8), device=dev)
    va, vb, vo = big[1:1 + n], big[n + 9:2 * n + 9], big[2 * n + 18:3 * n + 18]
    va.copy_(torch.from_numpy(a))
    vb.copy_(torch.from_numpy(b))
    ops.pseudo_gradient_(vo, va, vb, 2.0)
    assert np.array_equal(vo.cpu().numpy(), oracle.pseudo_gradient(a, b, 2.0))


@pytest.mark.parametrize("n", [1, 7, 4099, 2_000_001])
def test_outer_step_kernel_is_torch_sgd_nesterov(dev, oracle, n):
    from prime_amd import ops

    rng = np.random.default_rng(n + 1)
    p0 = rng.standard_normal(n).astype(np.float32)
    lr, mu = 0.7, 0.9
    cpu_p = torch.nn.Parameter(torch.from_numpy(p0.copy()))
    opt = torch.optim.SGD([cpu_p], lr=lr, momentum=mu, nesterov=True)        # diloco.py:72-74
    want_p, want_buf = p0.copy(), np.zeros(n, np.float32)
    gp = torch.from_numpy(p0.copy()).to(dev)
    gbuf = torch.zeros(n, device=dev)
    inner = torch.empty(n, device=dev)
    announce(f"outer step n={n}")
    for step in range(3):
        g = (rng.standard_normal(n) * 1e-2).astype(np.float32)
        cpu_p.grad = torch.from_numpy(g.copy())
        opt.step()
        oracle.outer_sgd_nesterov(want_p, want_buf, g, lr, mu, first_step=(step == 0))
        ops.outer_sgd_nesterov_(gp, gbuf, torch.from_numpy(g).to(dev), inner, lr, mu, step == 0)
        assert np.array_equal(gp.cpu().numpy(), want_p)
        assert np.array_equal(gp.cpu().numpy(), cpu_p.detach().numpy())
        assert np.array_equal(gbuf.cpu().numpy(), want_buf)
        assert torch.equal(inner, gp)


@pytest.mark.parametrize("n", [3, 65537, 1 << 20])
def test_outer_step_from_codes_equals_dequantize_then_step(dev, n):
    from prime_amd import ops

    g = torch.Generator(device=dev).manual_seed(n)
    grad = torch.randn(n, device=dev, generator=g) * 1e-3
    codes, lut = ops.uniform_8bit_quantize(grad)
    p1 = torch.randn(n, device=dev, generator=g)
    p2 = p1.clone()
    b1 = torch.randn(n, device=dev, generator=g) * 1e-3
    b2 = b1.clone()
    i1, i2 = torch.empty(n, device=dev), torch.empty(n, device=dev)
    announce(f"outer step from codes n={n}")
    for first in (True, False):
        ops.outer_sgd_nesterov_(p1, b1, ops.dequantize(codes, lut), i1, 0.7, 0.9, first)
        ops.outer_sgd_nesterov_codes_(p2, b2, codes, lut, i2, 0.7, 0.9, first)
        assert torch.equal(p1, p2) and torch.equal(b1, b2) and torch.equal(i1, i2)
    ops.outer_sgd_nesterov_codes_(p2, b2, codes, lut, None, 0.7, 0.9, False)       # no copy to an inner model
    ops.outer_sgd_nesterov_(p1, b1, ops.dequantize(codes, lut), None, 0.7, 0.9, False)
    assert torch.equal(p1, p2)


@pytest.mark.parametrize("shift", [1, 2, 3])
def test_outer_step_kernels_on_element_aligned_views(dev, oracle, shift):
    # parameters of a model are views at arbitrary element offsets of the flat buffers: the
    # element-aligned variants of both outer-step kernels against the oracle (itself pinned on torch's SGD)
    from prime_amd import ops

    n = 100_003
    rng = np.random.default_rng(shift)
    p0 = rng.standard_normal(n).astype(np.float32)
    b0 = (rng.standard_normal(n) * 1e-3).astype(np.float32)
    g0 = (rng.standard_normal(n) * 1e-3).astype(np.float32)
    pad = 16
    bufs = [torch.zeros(n + pad, device=dev) for _ in range(4)]
    p, b, g, inner = (t[shift + k:shift + k + n] for k, t in enumerate(bufs))
    p.copy_(torch.from_numpy(p0)); b.copy_(torch.from_numpy(b0)); g.copy_(torch.from_numpy(g0))
    announce(f"outer step misaligned shift={shift}")
    ops.outer_sgd_nesterov_(p, b, g, inner, 0.7, 0.9, False)
    wp, wb = p0.copy(), b0.copy()
    oracle.outer_sgd_nesterov(wp, wb, g0, 0.7, 0.9, first_step=False)
    assert np.array_equal(p.cpu().numpy(), wp) and np.array_equal(b.cpu().numpy(), wb) and torch.equal(inner, p)
    for t, lo in zip(bufs, (shift, shift + 1, shift + 2, shift + 3)):
        assert bool((t[:lo] == 0).all()) and bool((t[lo + n:] == 0).all())         # nothing written outside the views
    # from codes held in a byte buffer at an odd address
    codes, lut = ops.uniform_8bit_quantize(g)
    cbuf = torch.zeros(n + pad, dtype=torch.uint8, device=dev)
    cv = cbuf[shift:shift + n]
    cv.copy_(codes)
    ops.outer_sgd_nesterov_codes_(p, b, cv, lut, inner, 0.7, 0.9, False)
    deq = lut.cpu().numpy()[codes.cpu().numpy()]
    oracle.outer_sgd_nesterov(wp, wb, deq, 0.7, 0.9, first_step=False)
    assert np.array_equal(p.cpu().numpy(), wp) and np.array_equal(b.cpu().numpy(), wb) and torch.equal(inner, p)


def test_division_kernels_keep_denormals_like_the_cpu(dev, oracle):
    # pseudo-gradients of converged parameters can be denormal: (outer - inner) / W and chunk / W must round
    # as the CPU does, not flush to zero
    from prime_amd import ops

    rng = np.random.default_rng(0)
    n = 4099
    a = (rng.standard_normal(n) * 1e-38).astype(np.float32)
    b = (rng.standard_normal(n) * 1e-38).astype(np.float32)
    a[:8] = [1e-38, 3e-39, 1e-45, 0, -0.0, 2e-38, 1.1754944e-38, -1e-44]
    b[:8] = [0, 1e-39, 0, 0, 0, 1e-38, 1e-45, 1e-45]
    announce("denormal division")
    for W in (2.0, 3.0, 8.0, 14.0):
        out = torch.empty(n, device=dev)
        ops.pseudo_gradient_(out, torch.from_numpy(a).to(dev), torch.from_numpy(b).to(dev), W)
        want = oracle.pseudo_gradient(a, b, W)
        assert (np.abs(want) < 1.1754944e-38).sum() > n // 2 and np.count_nonzero(want) > n // 2
        assert np.array_equal(out.cpu().numpy().view(np.uint32), want.view(np.uint32))
        t = torch.from_numpy(a.copy()).to(dev)
        ops.div_(t, W)
        w2 = a.copy()
        oracle.div_scalar(w2, W)
        assert np.array_equal(t.cpu().numpy().view(np.uint32), w2.view(np.uint32))


class TinyLlama(nn.Module):
    """Parameter names shaped like the reference model's (layers.<i>.*), so the layer bucketing of
    get_offloaded_param (diloco.py:165-167) has something to group."""

    def __init__(self, d=64, layers=3):
        super().__init__()
        self.tok_embeddings = nn.Embedding(256, d)
        self.layers = nn.ModuleList([nn.ModuleDict({"wq": nn.Linear(d, d, bias=False), "w1": nn.Linear(d, 2 * d, bias=False),
                                                    "norm": nn.LayerNorm(d)}) for _ in range(layers)])
        self.output = nn.Linear(d, 256, bias=False)


def test_bucketing_follows_the_first_number_in_parameter_names(dev):
    from prime_amd.diloco import Diloco, _find_first_number

    assert _find_first_number("layers.12.attention.wq.weight") == 12 and _find_first_number("tok_embeddings.weight") == -1
    model = TinyLlama().to(dev)
    d = Diloco(0.7, model)
    names = [n for n, _ in model.named_parameters()]
    want, prev = [], None
    for n, p in model.named_parameters():
        if _find_first_number(n) != prev:
            want.append(0)
            prev = _find_first_number(n)
        want[-1] += p.numel()
    assert [b.numel() for b in d.grad_buckets] == want and len(want) == 5        # embeddings, 3 layers, output
    assert sum(want) == d.grad_flat.numel() == sum(p.numel() for p in model.parameters())
    assert names[0].startswith("tok_embeddings")


def test_outer_step_of_simulated_workers_against_cpu_emulation(dev, oracle):
    # W workers drift apart, then one DiLoCo outer step: GPU path against the reference's recipe on the
    # CPU (torch for the subtraction, the division and SGD; the oracle's ring for the all-reduce)
    from prime_amd.diloco import Diloco, step_simulated_workers

    W = 2
    torch.manual_seed(0)
    base = TinyLlama()
    models = [TinyLlama().to(dev) for _ in range(W)]
    for m in models:
        m.load_state_dict(base.state_dict())
    workers = [Diloco(0.7, m) for m in models]
    cpu_outer = [p.detach().clone() for p in base.parameters()]
    cpu_opt = torch.optim.SGD([nn.Parameter(p) for p in cpu_outer], lr=0.7, momentum=0.9, nesterov=True)
    cpu_params = [g["params"] for g in cpu_opt.param_groups][0]
    for outer in range(2):
        gen = torch.Generator().manual_seed(100 + outer)
        inner_cpu = []
        for r, m in enumerate(models):                       # the "inner steps": each worker moves on its own
            ps = []
            for p in m.parameters():
                delta = torch.randn(p.shape, generator=gen) * 1e-3
                p.data.add_(delta.to(dev))
                ps.append(p.detach().cpu().clone())
            inner_cpu.append(ps)
        announce(f"simulated diloco outer step {outer}")
        step_simulated_workers(workers, models)
        torch.cuda.synchronize()
        # CPU emulation: per worker grad = (outer - inner) / W, ring all-reduce per bucket, SGD step
        flat = [torch.cat([((o.detach() - i) / W).reshape(-1) for o, i in zip(cpu_params, inner_cpu[r])]).numpy().copy()
                for r in range(W)]
        lo = 0
        for b in workers[0].grad_buckets:
            n = b.numel()
            chunks = [f[lo:lo + n] for f in flat]
            oracle.ring_allreduce_sim(chunks)
            lo += n
        off = 0
        for p in cpu_params:
            p.grad = torch.from_numpy(flat[0][off:off + p.numel()].copy()).view(p.shape)
            off += p.numel()
        cpu_opt.step()
        for m in models:
            for gp, cp in zip(m.parameters(), cpu_params):
                # the ring is lossy (bins of ~1e-5 here) and its lookup tables differ in the last bits
                # between the two implementations, which moves a few elements that sit on a bin
                # boundary by one bin; everything else agrees to rounding
                diff = (gp.detach().cpu() - cp.detach()).abs()
                assert float(diff.max()) < 6e-5 and float(diff.mean()) < 3e-6
        for w in workers:                                   # outer copies equal the inner model after the step
            assert torch.equal(torch.cat([p.detach().reshape(-1) for p in models[0].parameters()]),
                               workers[0].outer_data_flat)
    # every worker holds the same model up to the ring's requantization on the all-gather path
    a = torch.cat([p.detach().reshape(-1) for p in models[0].parameters()])
    b = torch.cat([p.detach().reshape(-1) for p in models[1].parameters()])
    assert float((a - b).abs().max()) < 1e-4


@pytest.mark.parametrize("n,with_msg,divisor", [(1, False, 1.0), (4099, False, 1.0), (1 << 20, False, 1.0),
                                                (5, True, 1.0), (4099, True, 3.0), (1 << 20, True, 1.0), (3_000_001, True, 8.0)])
def test_ring_first_touch_is_pseudo_gradient_then_ring_step(dev, oracle, n, with_msg, divisor):
    # grad = (outer - inner) / W (diloco.py:93-101), [grad = (grad + lut[codes]) / divisor
    # (collectives.cpp:128-133, :155-159)], then uniform_8bit_quantize(grad): through the C ABI,
    # against the oracle and against the separate entry points
    from prime_amd import _lib
    from tests.conftest import lut_rel_err
    from tests.gpu_util import Abi

    abi = Abi(dev)
    rng = np.random.default_rng(n + 17)
    W = 4.0
    outer = rng.standard_normal(n).astype(np.float32)
    inner = (outer + rng.standard_normal(n).astype(np.float32) * 1e-3).astype(np.float32)
    announce(f"first touch n={n} msg={with_msg} divisor={divisor}")
    want = oracle.pseudo_gradient(outer, inner, W)
    codes_in = lut_in = None
    if with_msg:
        codes_in, lut_in, _ = abi.uniform(abi.to_dev((rng.standard_normal(n) * 2.5e-4).astype(np.float32)))
        oracle.index_add(want, lut_in.cpu().numpy(), codes_in.cpu().numpy())
        oracle.div_scalar(want, divisor)
    to, ti = abi.to_dev(outer), abi.to_dev(inner)
    grad = torch.full((n,), 7.0, device=dev)                         # overwritten entirely
    codes = torch.empty(n, dtype=torch.uint8, device=dev)
    lut = torch.empty(256, device=dev)
    qp = torch.empty(4, dtype=torch.float64, device=dev)
    _lib.check(abi.lib.prime_ring_first_touch(to.data_ptr(), ti.data_ptr(), n, W,
                                              codes_in.data_ptr() if with_msg else None, lut_in.data_ptr() if with_msg else None,
                                              divisor, grad.data_ptr(), codes.data_ptr(), lut.data_ptr(), qp.data_ptr(),
                                              abi.ws.data_ptr(), abi.st), "first touch")
    # the separate entry points
    g2 = torch.empty(n, device=dev)
    _lib.check(abi.lib.prime_pseudo_gradient_f32(to.data_ptr(), ti.data_ptr(), n, W, g2.data_ptr(), abi.st), "pg")
    if with_msg:
        abi.dequant(g2, lut_in, codes_in, add=True)
        _lib.check(abi.lib.prime_div_f32(g2.data_ptr(), n, divisor, abi.st), "div")
    codes2, lut2, qp2 = abi.uniform(g2)
    torch.cuda.synchronize()
    assert np.array_equal(grad.cpu().numpy(), want)
    assert np.array_equal(g2.cpu().numpy(), want)
    q = abi.qparams(qp)
    assert np.array_equal(np.array([q["scale"]]), np.array([oracle.scale_exact(want)]), equal_nan=True)
    oc, _, _ = oracle.uniform_8bit_quantize(want, "given", scale=float(q["scale"]))
    assert np.array_equal(codes.cpu().numpy(), oc)
    assert torch.equal(codes, codes2)
    mean, _ = oracle.average_buckets_f64(want, oc)
    floor = float(q["scale"]) if np.isfinite(q["scale"]) and q["scale"] > 0 else 1.0
    assert lut_rel_err(lut.cpu().numpy(), mean, floor) <= 1e-6
    assert np.array_equal(to.cpu().numpy(), outer) and np.array_equal(ti.cpu().numpy(), inner)


def test_ring_first_touch_rejects_bad_arguments(dev):
    from prime_amd import ops

    n = 64
    o, i, g = (torch.zeros(n, device=dev) for _ in range(3))
    codes = torch.zeros(n, dtype=torch.uint8, device=dev)
    lut = torch.zeros(256, device=dev)
    with pytest.raises(RuntimeError, match="together"):
        ops.ring_first_touch_(g, o, i, 2.0, codes, None, 1.0)
    with pytest.raises(RuntimeError, match="divisor"):
        ops.ring_first_touch_(g, o, i, 2.0, None, None, 2.0)
    with pytest.raises(RuntimeError, match="divisor"):
        ops.ring_first_touch_(g, o, i, 2.0, codes, lut, 0.0)
    with pytest.raises(RuntimeError, match="numel"):
        ops.ring_first_touch_(g, o, i, 2.0, codes[:8], lut, 1.0)


@pytest.mark.parametrize("W", [1, 2, 4])
def test_flat_inner_workers_with_lazy_pseudo_gradient_equal_the_plain_ones(dev, W):
    # same arithmetic, fewer passes: with the model's parameters in one flat buffer the ring forms
    # each chunk's pseudo-gradient on its first visit; parameters after two outer steps must equal
    # those of workers that materialize the pseudo-gradient first, bit for bit
    from prime_amd.diloco import Diloco, step_simulated_workers

    torch.manual_seed(1)
    base = TinyLlama()
    plain = [TinyLlama().to(dev) for _ in range(W)]
    flat = [TinyLlama().to(dev) for _ in range(W)]
    for m in plain + flat:
        m.load_state_dict(base.state_dict())
    wp = [Diloco(0.7, m) for m in plain]
    wf = [Diloco(0.7, m, flat_inner=True) for m in flat]
    assert all(w._inner_is_flat(m) for w, m in zip(wf, flat))
    for outer in range(2):
        gen = torch.Generator().manual_seed(200 + outer)
        for mp, mf in zip(plain, flat):
            for p, f in zip(mp.parameters(), mf.parameters()):
                delta = (torch.randn(p.shape, generator=gen) * 1e-3).to(dev)
                p.data.add_(delta)
                f.data.add_(delta)
        announce(f"flat-inner diloco W={W} outer step {outer}")
        step_simulated_workers(wp, plain)
        step_simulated_workers(wf, flat, coded_gather=False)
        torch.cuda.synchronize()
        for mp, mf, w in zip(plain, flat, wf):
            assert w._inner_is_flat(mf)
            for p, f in zip(mp.parameters(), mf.parameters()):
                assert torch.equal(p.detach(), f.detach())
        for a, b in zip(wp, wf):
            assert torch.equal(a.outer_data_flat, b.outer_data_flat) and torch.equal(a.momentum_flat, b.momentum_flat)
    # a model can still be used as a module: forward through the flat views
    y = flat[0].output(torch.randn(2, 64, device=dev))
    assert y.shape == (2, 256)


@pytest.mark.parametrize("W", [1, 2, 4])
def test_flat_inner_workers_with_coded_all_gather_track_the_plain_ones(dev, W):
    # the fastest arrangement: lazy pseudo-gradient, all-gather in the code domain, outer step straight
    # from codes.  Same codes everywhere; lookup entries of forwarded chunks agree to rounding only, so
    # parameters agree to rounding except where an element crossed a bin edge
    from prime_amd.diloco import Diloco, step_simulated_workers

    torch.manual_seed(2)
    base = TinyLlama()
    plain = [TinyLlama().to(dev) for _ in range(W)]
    flat = [TinyLlama().to(dev) for _ in range(W)]
    for m in plain + flat:
        m.load_state_dict(base.state_dict())
    wp = [Diloco(0.7, m) for m in plain]
    wf = [Diloco(0.7, m, flat_inner=True) for m in flat]
    for outer in range(2):
        gen = torch.Generator().manual_seed(300 + outer)
        for mp, mf in zip(plain, flat):
            for p, f in zip(mp.parameters(), mf.parameters()):
                delta = (torch.randn(p.shape, generator=gen) * 1e-3).to(dev)
                p.data.add_(delta)
                f.data.add_(delta)
        announce(f"coded diloco W={W} outer step {outer}")
        step_simulated_workers(wp, plain)
        step_simulated_workers(wf, flat)                  # coded_gather is the default
        torch.cuda.synchronize()
        for a, b, mf in zip(wp, wf, flat):
            assert b._inner_is_flat(mf) and not b._first_step
            assert torch.equal(b.inner_flat, b.outer_data_flat)
            diff = (a.outer_data_flat - b.outer_data_flat).abs()
            assert float(diff.max()) < 6e-5 and float(diff.mean()) < 3e-7
            assert float((a.momentum_flat - b.momentum_flat).abs().max()) < 6e-5


def test_uncompressed_simulated_all_reduce_and_fake_step(dev):
    from prime_amd.C.collectives import SimulatedRing
    from prime_amd.collectives import Compression, all_reduce
    from prime_amd.diloco import Diloco
    import torch.distributed as dist

    xs = [torch.full((8,), float(r + 1), device=dev) for r in range(3)]
    all_reduce(Compression.NO, xs[0], dist.ReduceOp.SUM, SimulatedRing(xs))
    assert all(bool((x == 6).all()) for x in xs)
    model = TinyLlama().to(dev)
    d = Diloco(0.7, model, compression=Compression.NO)
    before = [p.detach().clone() for p in model.parameters()]
    d.step(model, group=SimulatedRing([d.grad_flat]), world_size=1, fake=True)     # fake: zero pseudo-gradient (:95-96)
    for p, q in zip(model.parameters(), before):
        assert torch.equal(p.detach(), q)


def test_all_reduce_is_retried_and_falls_back_to_the_unreduced_pseudo_gradient(dev):
    # diloco.py:92-132: every attempt forms the pseudo-gradient afresh and all-reduces the buckets; an attempt that
    # raises is followed by another on the group regroup() returns; when all have failed the worker keeps
    # outer - inner, not divided by the world size
    from prime_amd.C.collectives import SimulatedRing
    from prime_amd.collectives import Compression
    from prime_amd.diloco import Diloco

    class Broken:
        """A group whose all-reduce cannot run: prime_amd.collectives.all_reduce raises on it."""

    torch.manual_seed(5)
    model = TinyLlama().to(dev)
    d = Diloco(0.7, model, compression=Compression.NO)
    for p in model.parameters():
        p.data.add_(torch.randn_like(p) * 1e-3)
    inner = torch.cat([p.detach().reshape(-1) for p in model.parameters()])
    want = d.outer_data_flat - inner

    # every attempt fails: the fallback
    calls = []
    ok = d.sync_pseudo_gradient(model, Broken(), world_size=4, retry_all_reduce=3, regroup=lambda: calls.append(1) or Broken())
    assert ok is False and len(calls) == 2 and d.last_all_reduce_error is not None
    assert torch.equal(d.grad_flat, want)                                   # not divided by 4

    # the second attempt succeeds on the group regroup() hands over: SUM over one simulated rank of grad / 4
    ok = d.sync_pseudo_gradient(model, Broken(), world_size=4, retry_all_reduce=3, regroup=lambda: SimulatedRing([d.grad_flat]))
    assert ok is True
    assert torch.equal(d.grad_flat, want / 4.0)

    # without retries the exception reaches the caller, as before
    with pytest.raises(Exception):
        d.step(model, group=Broken(), world_size=4)
    with pytest.raises(ValueError, match="at least 1"):
        d.sync_pseudo_gradient(model, Broken(), world_size=4, retry_all_reduce=0)

    # step() with retries applies the outer optimizer to the fallback gradient
    before = d.outer_data_flat.clone()
    d.step(model, group=Broken(), world_size=4, retry_all_reduce=2)
    torch.cuda.synchronize()
    # first Nesterov step: p -= lr (1 + mu) g; the difference of two fp32 parameters of size ~1 carries ~1e-7
    assert torch.allclose(before - d.outer_data_flat, 0.7 * 1.9 * want, rtol=1e-4, atol=1e-6)


def test_outer_step_with_a_real_process_group_of_one_rank(dev, oracle, tmp_path):
    # the reference's call site unchanged: all_reduce(Compression.UINT8, bucket, SUM, group) on the default
    # process group; with one rank no message is sent, but every bucket's two chunks still take the lossy
    # quantize / dequantize round trip (collectives.cpp:161-173)
    import torch.distributed as dist

    from prime_amd.collectives import Compression, all_reduce
    from prime_amd.diloco import Diloco

    assert not dist.is_initialized()
    dist.init_process_group("gloo", init_method=f"file://{tmp_path}/rendezvous", rank=0, world_size=1)
    try:
        rng = np.random.default_rng(8)
        x = (rng.standard_normal(40_000) * 1e-3).astype(np.float32)
        t = torch.from_numpy(x.copy()).to(dev)
        announce("one-rank process group: all_reduce")
        all_reduce(Compression.UINT8, t, dist.ReduceOp.SUM)              # group=None: the default group
        want = [x.copy()]
        oracle.ring_allreduce_sim(want)
        assert np.allclose(t.cpu().numpy(), want[0], rtol=2e-6, atol=1e-9)
        half = x.size // 2
        assert len(np.unique(t.cpu().numpy()[:half])) <= 256 and len(np.unique(t.cpu().numpy()[half:])) <= 256
        # a whole outer step of one worker through Diloco.step, world size taken from the group
        torch.manual_seed(3)
        model = TinyLlama().to(dev)
        d = Diloco(0.7, model)
        before = d.outer_data_flat.clone()
        for p in model.parameters():
            p.data.add_(torch.randn_like(p) * 1e-3)
        inner = torch.cat([p.detach().reshape(-1) for p in model.parameters()])
        announce("one-rank process group: Diloco.step")
        d.step(model)
        torch.cuda.synchronize()
        # first outer step of SGD with Nesterov momentum: p -= lr * (1 + mu) * g, with g the quantized (outer - inner)
        g_exact = before - inner
        moved = before - d.outer_data_flat
        err = (moved - 0.7 * 1.9 * g_exact).abs() / (0.7 * 1.9)
        bin_width = 6 * 1e-3 / 256                   # per bucket about this: 6 sigma over 256 bins
        assert float((err > 1.2 * bin_width).float().mean()) < 0.01        # all but the clipped tails (beyond 3 sigma)
        assert float(err.mean()) < 0.5 * bin_width
        assert torch.equal(torch.cat([p.detach().reshape(-1) for p in model.parameters()]), d.outer_data_flat)
    finally:
        dist.destroy_process_group()
