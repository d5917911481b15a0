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
