"""Segmented launches (many tensors, three kernel launches in all) against the one-tensor entry
points and the CPU oracle, through the C ABI.

Bar: tensor i's codes, lookup table and statistics record equal what the one-tensor entry point
returns for it, bit for bit; codes and tables are also held to the oracle as in test_gpu_parity.
"""
import numpy as np
import pytest
import torch

from tests.conftest import lut_rel_err
from tests.gpu_util import Abi, announce, segmented_ring_step, segmented_uniform

pytestmark = pytest.mark.gpu

LUT_TOL = 1e-6
RING_CHUNK_CFG2 = 51_380_224 // 16      # a 1B model's layer bucket cut into 2 * 8 chunks (collectives.cpp:89-90)
RING_CHUNK_CFG4 = 1_860_119             # a 10B model's shard bucket (29,761,904 elements) cut the same way, rounded down


@pytest.fixture(scope="module")
def abi(dev):
    return Abi(dev)


def bits(t: torch.Tensor) -> np.ndarray:
    return t.detach().cpu().contiguous().view(torch.uint8).numpy()


def mixed_tensors(rng):
    """Sizes from one element to a ring chunk, and the value patterns the one-tensor tests use."""
    out = {}
    out["ring chunk cfg2"] = (rng.standard_t(3, RING_CHUNK_CFG2) * 1e-4).astype(np.float32)
    out["ring chunk cfg4, odd size"] = (rng.standard_normal(RING_CHUNK_CFG4) * 5e-4).astype(np.float32)
    out["2^20"] = (rng.standard_normal(1 << 20) * 1e-3).astype(np.float32)
    out["2^20 constant"] = np.full(1 << 20, 0.25, np.float32)
    out["2^20 zeros"] = np.zeros(1 << 20, np.float32)
    half = (rng.standard_normal(1 << 20) * 1e-3).astype(np.float32)
    half[rng.random(1 << 20) < 0.5] = 0
    out["2^20 half zeros"] = half
    out["narrow N(1, 1e-2)"] = (rng.standard_normal(300_001) * 1e-2 + 1).astype(np.float32)
    outl = (rng.standard_normal(500_000) * 5e-4).astype(np.float32)
    pos = rng.choice(outl.size, 50, replace=False)
    outl[pos] = np.where(rng.random(50) < 0.5, -1, 1) * 50 * 5e-4
    out["outliers at 50 sigma"] = outl
    out["65543"] = (rng.standard_normal(65_543) * 1e-3).astype(np.float32)
    out["16384 (one launch on its own)"] = (rng.standard_normal(16_384) * 1e-3).astype(np.float32)
    out["4097"] = (rng.standard_normal(4_097) * 1e-3).astype(np.float32)
    out["5"] = (rng.standard_normal(5) * 1e-3).astype(np.float32)
    out["1"] = np.array([0.5], np.float32)
    return out


def test_segmented_uniform_equals_one_tensor_calls_and_oracle(abi, oracle):
    rng = np.random.default_rng(31)
    cases = mixed_tensors(rng)
    xs = [abi.to_dev(v) for v in cases.values()]
    announce(f"segmented uniform, {len(xs)} tensors, sizes {[x.numel() for x in xs]}")
    codes, luts, qps = segmented_uniform(abi, xs)
    torch.cuda.synchronize()
    for i, (label, x) in enumerate(cases.items()):
        announce(f"one-tensor call: {label}")
        c1, l1, q1 = abi.uniform(xs[i])
        torch.cuda.synchronize()
        assert np.array_equal(bits(qps[i]), bits(q1)), label
        assert np.array_equal(codes[i].cpu().numpy(), c1.cpu().numpy()), label
        assert np.array_equal(bits(luts[i]), bits(l1)), label
        # and the oracle
        q = abi.qparams(qps[i])
        assert np.array_equal(np.array([q["scale"]]), np.array([oracle.scale_exact(x)]), equal_nan=True), label
        if x.size > 1:
            oc, _, _ = oracle.uniform_8bit_quantize(x, "given", scale=float(q["scale"]))
            gc = codes[i].cpu().numpy()
            assert np.array_equal(gc, oc), label
            mean, cnt = oracle.average_buckets_f64(x, gc)
            floor = float(q["scale"]) if np.isfinite(q["scale"]) and q["scale"] > 0 else 1.0
            assert lut_rel_err(luts[i].cpu().numpy(), mean, floor) <= LUT_TOL, label


@pytest.mark.parametrize("kind", ["reduce", "gather", "reduce_div"])
def test_segmented_ring_step_equals_one_chunk_calls(abi, oracle, kind):
    # W = 8 ranks' chunks of a 1B model's layer bucket in one step of the lock-stepped ring, plus ragged ones
    rng = np.random.default_rng(32)
    sizes = [RING_CHUNK_CFG2] * 8 + [RING_CHUNK_CFG4, 1 << 20, 65_543, 16_384, 4_099, 7]
    accs_np = [(rng.standard_normal(n) * 1e-3).astype(np.float32) for n in sizes]
    msgs = []
    for n in sizes:
        src = abi.to_dev((rng.standard_normal(n) * 1e-3).astype(np.float32))
        c, l, _ = abi.uniform(src)
        msgs.append((c, l))
    divisor = 8.0 if kind == "reduce_div" else 1.0
    accs = [abi.to_dev(a) for a in accs_np]
    announce(f"segmented ring {kind} step, sizes {sizes}")
    codes, luts, qps = segmented_ring_step(abi, kind, accs, [m[0] for m in msgs], [m[1] for m in msgs], divisor)
    torch.cuda.synchronize()
    for i, n in enumerate(sizes):
        announce(f"one-chunk {kind} step n={n}")
        acc1 = abi.to_dev(accs_np[i])
        c1, l1, q1 = abi.ring_step(acc1, msgs[i][0], msgs[i][1], gather=kind == "gather",
                                   divisor=divisor if kind == "reduce_div" else None)
        torch.cuda.synchronize()
        assert np.array_equal(bits(accs[i]), bits(acc1)), (kind, n)
        assert np.array_equal(bits(qps[i]), bits(q1)), (kind, n)
        assert np.array_equal(codes[i].cpu().numpy(), c1.cpu().numpy()), (kind, n)
        assert np.array_equal(bits(luts[i]), bits(l1)), (kind, n)
    # the first chunk against the oracle (collectives.cpp:128-138 / :204-215 / :155-162)
    c_in, l_in = msgs[0][0].cpu().numpy(), msgs[0][1].cpu().numpy()
    want = accs_np[0].copy()
    if kind == "gather":
        oracle.index_set(want, l_in, c_in)
    else:
        oracle.index_add(want, l_in, c_in)
        if kind == "reduce_div":
            oracle.div_scalar(want, divisor)
    assert np.array_equal(accs[0].cpu().numpy(), want)
    q = abi.qparams(qps[0])
    assert q["scale"] == oracle.scale_exact(want)
    oc, _, _ = oracle.uniform_8bit_quantize(want, "given", scale=float(q["scale"]))
    assert np.array_equal(codes[0].cpu().numpy(), oc)
    mean, _ = oracle.average_buckets_f64(want, oc)
    assert lut_rel_err(luts[0].cpu().numpy(), mean, float(q["scale"])) <= LUT_TOL


def test_segmented_call_takes_empty_and_misaligned_tensors_and_more_than_one_group(abi, oracle):
    rng = np.random.default_rng(33)
    base = abi.to_dev((rng.standard_normal(300_000) * 1e-3).astype(np.float32))
    xs = [base[1:100_001],                                  # starts at an odd element: not 16-byte aligned
          torch.empty(0, dtype=torch.float32, device=abi.dev),
          base[100_004:200_004]]
    xs += [abi.to_dev((rng.standard_normal(int(n)) * 1e-3).astype(np.float32)) for n in rng.integers(1, 40_000, 70)]
    announce(f"segmented uniform with an empty and a misaligned tensor, {len(xs)} tensors")
    codes, luts, qps = segmented_uniform(abi, xs)
    torch.cuda.synchronize()
    for i, x in enumerate(xs):
        c1, l1, q1 = abi.uniform(x.contiguous() if x.numel() == 0 else x)
        torch.cuda.synchronize()
        if x.numel():
            assert np.array_equal(bits(qps[i]), bits(q1)), i
        assert np.array_equal(codes[i].cpu().numpy(), c1.cpu().numpy()), i
        assert np.array_equal(bits(luts[i]), bits(l1)), i


def test_segmented_ops_layer(dev, oracle):
    # the torch-facing wrappers (prime_amd.ops.SegmentPlan and friends) against the one-tensor ops
    from prime_amd import ops

    g = torch.Generator(device=dev).manual_seed(34)
    xs = [torch.randn(n, device=dev, generator=g) * 1e-3 for n in (200_000, 1 << 20, 70_001, 12)]
    codes, luts = ops.uniform_8bit_quantize_segmented(xs)
    for x, c, l in zip(xs, codes, luts):
        c1, l1 = ops.uniform_8bit_quantize(x, False)
        assert torch.equal(c, c1) and np.array_equal(bits(l), bits(l1))
    accs = [torch.randn(x.numel(), device=dev, generator=g) * 1e-3 for x in xs]
    accs1 = [a.clone() for a in accs]
    codes2, luts2 = ops.ring_step_segmented(ops.SEG_REDUCE, accs, codes, list(luts))
    for a, a1, c_in, l_in, c, l in zip(accs, accs1, codes, luts, codes2, luts2):
        c1, l1 = ops.ring_reduce_step(a1, c_in, l_in)
        assert torch.equal(a, a1) and torch.equal(c, c1) and np.array_equal(bits(l), bits(l1))


def test_segmented_pointwise_passes_equal_the_one_tensor_calls(dev, oracle):
    # the per-parameter loops of diloco.py:93-99 and :212-215 as one launch per 64 tensors: 150 parameter-like
    # tensors, among them empty ones, one of three elements and views that start at an odd element
    from prime_amd import ops

    rng = np.random.default_rng(35)
    g = torch.Generator(device=dev).manual_seed(35)
    sizes = [int(n) for n in rng.integers(1, 300_000, 146)] + [0, 3, 1 << 21, 0]
    pool = torch.randn(sum(sizes) + 8, device=dev, generator=g)

    def views(shift):
        out, off = [], shift
        for n in sizes:
            out.append(pool[off:off + n])
            off += n
        return out

    for shift in (0, 1):                      # shift 1: most views are not 16-byte aligned
        outers = views(shift)
        inners = [o + torch.randn(o.numel(), device=dev, generator=g) * 1e-3 for o in outers]
        grads = [torch.empty_like(o) for o in outers]
        announce(f"segmented pseudo-gradient, {len(sizes)} tensors, shift {shift}")
        ops.pseudo_gradient_segmented_(grads, outers, inners, 4.0)
        for o, i, gr in zip(outers, inners, grads):
            want = torch.empty_like(o)
            if o.numel():
                ops.pseudo_gradient_(want, o, i, 4.0)
            assert np.array_equal(bits(gr), bits(want))
            assert np.array_equal(gr.cpu().numpy(), oracle.pseudo_gradient(o.cpu().numpy(), i.cpu().numpy(), 4.0))
        for first in (True, False):
            params = [o.clone() for o in outers]
            moms = [torch.randn(o.numel(), device=dev, generator=g) for o in outers]
            models = [torch.empty_like(o) for o in outers]
            p1 = [p.clone() for p in params]
            m1 = [m.clone() for m in moms]
            i1 = [torch.empty_like(o) for o in outers]
            announce(f"segmented outer step, first_step={first}, shift {shift}")
            ops.outer_sgd_nesterov_segmented_(params, moms, grads, models, 0.7, 0.9, first)
            for k in range(len(sizes)):
                if sizes[k]:
                    ops.outer_sgd_nesterov_(p1[k], m1[k], grads[k], i1[k], 0.7, 0.9, first)
                    assert np.array_equal(bits(params[k]), bits(p1[k])) and np.array_equal(bits(moms[k]), bits(m1[k]))
                    assert np.array_equal(bits(models[k]), bits(i1[k]))
        # without an inner model
        params = [o.clone() for o in outers]
        moms = [torch.zeros_like(o) for o in outers]
        p1 = [p.clone() for p in params]
        ops.outer_sgd_nesterov_segmented_(params, moms, grads, None, 0.7, 0.9, True)
        for k in range(len(sizes)):
            if sizes[k]:
                m = torch.zeros_like(p1[k])
                ops.outer_sgd_nesterov_(p1[k], m, grads[k], None, 0.7, 0.9, True)
                assert np.array_equal(bits(params[k]), bits(p1[k]))


def test_batched_op_routes_a_set_with_a_large_entry_through_the_segmented_call(dev):
    # prime::uniform_8bit_quantize_batched gives every tensor one workgroup; with host-visible offsets a set that
    # holds an entry of more than 65,536 elements takes the segmented path instead: same results as tensor by tensor
    from prime_amd import _lib, ops

    g = torch.Generator(device=dev).manual_seed(36)
    sizes = [5_000, 300_000, 0, 12, 70_000]
    flat = torch.randn(sum(sizes), device=dev, generator=g) * 1e-3
    off = torch.tensor(np.concatenate([[0], np.cumsum(sizes)]), dtype=torch.int64)        # on the host
    _lib.profile_begin()
    codes, luts, qps = ops.uniform_8bit_quantize_batched(flat, off)
    kernels = _lib.profile_end()
    assert "batched_kernel" not in kernels and "seg_quantize_kernel+hist" in kernels
    bounds = off.tolist()
    for t, (a, b) in enumerate(zip(bounds, bounds[1:])):
        c1, l1, q1 = ops.uniform_8bit_quantize_stats(flat[a:b])
        assert torch.equal(codes[a:b], c1) and np.array_equal(bits(luts[t]), bits(l1))
        if b > a:
            assert np.array_equal(bits(qps[t]), bits(q1))
    with pytest.raises(RuntimeError, match="non-decreasing"):
        ops.uniform_8bit_quantize_batched(flat, torch.tensor([0, 10, 5], dtype=torch.int64))
    # small entries only: the one-launch kernel, as before
    off2 = torch.tensor([0, 100, 4000, 4000, 60_000], dtype=torch.int64)
    _lib.profile_begin()
    ops.uniform_8bit_quantize_batched(flat, off2)
    assert list(_lib.profile_end()) == ["batched_kernel"]
