"""Pins the CPU oracle (oracle/prime_oracle.cpp) before anything is compared against it.

Every check here is independent of the oracle's own formula: closed forms, the reference
test's own vector, brute force over float neighbourhoods of every bin boundary, exact
integer arithmetic, libtorch's norm, the fixtures written by the compiled reference, and
(when it has been built) the compiled reference itself.
"""
import math

import numpy as np
import pytest

from tests.golden.make_fixtures import CASES, case_input


# ---------------------------------------------------------------- quantize (compression.cpp:9-43)

def test_quantize_power_of_two_scale_closed_form(oracle):
    # x = m * 2^-k is exact, so x * (1/scale) == m exactly and code == clamp(m + 128)
    for k in (0, 3, 10, 20):
        scale = 2.0 ** -k
        m = np.arange(-300, 301, dtype=np.float32)
        codes = oracle.quantize_per_tensor_uint8(m * np.float32(scale), scale, 128)
        assert np.array_equal(codes, np.clip(m.astype(np.int64) + 128, 0, 255).astype(np.uint8))


def test_quantize_ties_round_away_from_zero(oracle):
    # (m + 1/2) * scale is a tie: std::round goes away from zero (half-even would give evens)
    m = np.arange(-100, 100, dtype=np.float32)
    x = (m + 0.5) * np.float32(0.25)
    codes = oracle.quantize_per_tensor_uint8(x, 0.25, 128).astype(np.int64) - 128
    want = np.where(m + 0.5 > 0, m + 1, m).astype(np.int64)
    assert np.array_equal(codes, want)


def test_quantize_reference_test_vector(oracle, golden):
    # tests/test_c/test_compression.py:46-48: ones * 10, scale 0.01, zero point 128 -> saturates
    codes = oracle.quantize_per_tensor_uint8(np.full(1000, 10.0, np.float32), 0.01, 128)
    assert (codes == 255).all()
    assert np.array_equal(codes, golden["qpt_ones/codes"])


def test_quantize_zero_point_other_than_128(oracle):
    x = np.array([-3.0, -1.0, 0.0, 1.0, 3.0, 300.0], np.float32)
    assert list(oracle.quantize_per_tensor_uint8(x, 1.0, 0)) == [0, 0, 0, 1, 3, 255]
    assert list(oracle.quantize_per_tensor_uint8(x, 1.0, 250)) == [247, 249, 250, 251, 253, 255]


def test_quantize_special_values_follow_x86_conversion(oracle):
    # NaN, +-inf and anything beyond int32 convert to INT_MIN on x86 and so land on code 0,
    # +inf included; 2^31 - 128 + 128 wraps
    x = np.array([np.nan, np.inf, -np.inf, 3e38, -3e38, 2147483520.0, 2147483648.0, -2147483648.0,
                  2147483392.0, 1e-40, -1e-40], np.float32)
    assert list(oracle.quantize_per_tensor_uint8(x, 1.0, 128)) == [0, 0, 0, 0, 0, 0, 0, 0, 255, 128, 128]


def test_quantize_brute_force_around_every_boundary(oracle):
    # For a non-trivial inv_scale, walk the floats on either side of every bin boundary and
    # compare with round-half-away computed in exact rational arithmetic on the fp32 product.
    scale = np.float32(2.3418523e-05)
    inv = np.float32(1.0) / scale
    xs = []
    for k in range(-130, 130):
        centre = np.float32((k + 0.5) * float(scale))
        v = centre
        for _ in range(40):
            v = np.nextafter(v, np.float32(-np.inf), dtype=np.float32)
        for _ in range(80):
            xs.append(v)
            v = np.nextafter(v, np.float32(np.inf), dtype=np.float32)
    x = np.array(xs, np.float32)
    prod = (x * inv).astype(np.float32)            # one fp32 multiply, as compression.cpp:23
    p64 = prod.astype(np.float64)
    r = np.where(p64 >= 0, np.floor(p64 + 0.5), np.ceil(p64 - 0.5))
    want = np.clip(r.astype(np.int64) + 128, 0, 255).astype(np.uint8)
    got = oracle.quantize_per_tensor_uint8(x, float(scale), 128)
    assert np.array_equal(got, want)
    assert len(np.unique(got)) == 256


def test_quantize_thread_slicing_does_not_change_result(oracle):
    x = (np.random.default_rng(3).standard_normal(10007) * 3).astype(np.float32)
    base = oracle.quantize_per_tensor_uint8(x, 0.05, 128, threads=1)
    for t in (2, 3, 8, 64):
        assert np.array_equal(base, oracle.quantize_per_tensor_uint8(x, 0.05, 128, threads=t))


def test_quantize_matches_reference_fixtures(oracle, golden):
    x = case_input("normal:4096") * 1000.0
    for i in range(5):
        scale = float(golden[f"qpt_{i}/scale"][0])
        assert np.array_equal(oracle.quantize_per_tensor_uint8(x, scale, 128), golden[f"qpt_{i}/codes"])


# ---------------------------------------------------------------- average_buckets (compression.cpp:45-104)

def test_average_buckets_integer_values_are_exact(oracle):
    # small integers: every partial sum is exact in fp32, so any summation order gives the same bits
    rng = np.random.default_rng(11)
    x = rng.integers(-50, 50, 200000).astype(np.float32)
    codes = rng.integers(0, 256, 200000).astype(np.uint8)
    for t in (1, 8):
        lut, cnt = oracle.average_buckets(x, codes, 256, threads=t, return_counts=True)
        assert np.array_equal(cnt, np.bincount(codes, minlength=256))
        sums = np.bincount(codes, weights=x.astype(np.float64), minlength=256)
        want = (sums.astype(np.float32) / cnt.astype(np.float32)).astype(np.float32)
        assert np.array_equal(lut, want)


def test_average_buckets_empty_bin_is_zero_and_small_n_bins_skips(oracle):
    x = np.array([1.0, 2.0, 3.0, 5.0], np.float32)
    codes = np.array([0, 0, 3, 200], np.uint8)
    lut = oracle.average_buckets(x, codes, 256)
    assert lut[0] == 1.5 and lut[3] == 3.0 and lut[200] == 5.0 and lut[1] == 0.0 and lut.sum() == 9.5
    lut8 = oracle.average_buckets(x, codes, 8)      # code 200 >= n_bins is skipped (:70)
    assert lut8.shape == (8,) and lut8[0] == 1.5 and lut8[3] == 3.0


def test_average_buckets_f64_is_bincount(oracle):
    rng = np.random.default_rng(5)
    x = (rng.standard_normal(50000) * 10).astype(np.float32)
    codes = rng.integers(0, 255, 50000).astype(np.uint8)
    mean, cnt = oracle.average_buckets_f64(x, codes)
    sums = np.bincount(codes, weights=x.astype(np.float64), minlength=256)
    c = np.bincount(codes, minlength=256)
    want = np.where(c > 0, sums / np.maximum(c, 1), 0.0)
    assert np.array_equal(cnt, c)
    assert np.allclose(mean, want, rtol=1e-13, atol=0)


def test_average_buckets_matches_reference_fixture(oracle, golden):
    from tests.conftest import lut_rel_err

    lut = oracle.average_buckets(golden["avg/x"], golden["avg/codes"], 256)
    # the reference's own sums are fp32 and thread-order dependent: agree to fp32 noise
    assert lut_rel_err(lut, golden["avg/lut"].astype(np.float64), 1e-3) < 2e-5
    mean, _ = oracle.average_buckets_f64(golden["avg/x"], golden["avg/codes"])
    assert lut_rel_err(golden["avg/lut"], mean, 1e-3) < 2e-5
    assert golden["avg/lut"][255] == 0.0            # randint(0, 255) never draws 255: empty bin


# ---------------------------------------------------------------- scale and the whole op (compression.cpp:106-125)

def test_norm_literal_matches_libtorch(oracle):
    import torch

    rng = np.random.default_rng(1)
    for n in list(range(1, 40)) + [100, 255, 1000, 4099, 65536, 65543, (1 << 20) + 5]:
        x = (rng.standard_normal(n) * 1e-3).astype(np.float32)
        assert oracle.norm_literal(x) == np.float32(torch.from_numpy(x).norm().item()), n


def test_scale_formula_closed_form(oracle):
    # all ones: sum of squares = n exactly; scale = 6 * sqrt(n) / sqrt(n-1) / 256
    for n in (2, 5, 4096, 1 << 20):
        want = np.float32(6.0 * (float(np.float32(math.sqrt(n))) / math.sqrt(n - 1)) / 256.0)
        assert oracle.scale_exact(np.ones(n, np.float32)) == want
        assert oracle.scale_from_norm(float(np.float32(math.sqrt(n))), n) == want


def test_stats_f64_against_integer_arithmetic(oracle):
    rng = np.random.default_rng(2)
    xi = rng.integers(-1000, 1000, 1 << 20)
    s, q = oracle.stats_f64(xi.astype(np.float32))
    assert s == float(xi.sum()) and q == float((xi.astype(np.int64) ** 2).sum())


def test_uniform_constant_tensor_is_code_171(oracle):
    # every element c > 0: x / scale = 256 / 6 * sqrt((n-1)/n) -> 42.67 -> 43 + 128 = 171
    for norm in ("exact", "literal"):
        codes, lut, _ = oracle.uniform_8bit_quantize(np.full(5000, 0.25, np.float32), norm)
        assert (codes == 171).all()
        assert lut[171] == np.float32(0.25) and np.count_nonzero(lut) == 1


def test_uniform_zero_tensor_and_single_element(oracle):
    # zeros: scale 0 -> inv = inf -> 0 * inf = NaN -> code 0; lookup all zero
    codes, lut, scale = oracle.uniform_8bit_quantize(np.zeros(100, np.float32), "exact")
    assert scale == 0.0 and (codes == 0).all() and not lut.any()
    # n = 1: std = norm / sqrt(0) = inf -> inv = 0 -> code 128, lut[128] = x
    codes, lut, scale = oracle.uniform_8bit_quantize(np.array([0.7], np.float32), "exact")
    assert np.isinf(scale) and codes[0] == 128 and lut[128] == np.float32(0.7)
    # n = 1, x = 0: 0 / 0 = NaN scale -> code 0
    codes, lut, scale = oracle.uniform_8bit_quantize(np.zeros(1, np.float32), "exact")
    assert np.isnan(scale) and codes[0] == 0 and not lut.any()


def test_uniform_invariants(oracle):
    x = (np.random.default_rng(0).standard_normal(1 << 18) * 1e-3).astype(np.float32)
    codes, lut, scale = oracle.uniform_8bit_quantize(x, "exact")
    mean, cnt = oracle.average_buckets_f64(x, codes)
    assert cnt.sum() == x.size
    assert abs((cnt * mean).sum() - x.astype(np.float64).sum()) < 1e-9
    inside = (codes > 0) & (codes < 255)
    assert np.abs(x[inside] - lut[codes[inside]]).max() <= scale
    filled = lut[cnt > 0]
    assert (np.diff(filled) > 0).all()
    # 6-sigma range over 256 bins: scale ~= 6 sigma / 256
    assert abs(scale / (6 * 1e-3 / 256) - 1) < 0.01


@pytest.mark.parametrize("name", CASES)
def test_uniform_matches_reference_fixtures(oracle, golden, name):
    from tests.conftest import lut_rel_err

    key = name.replace(":", "_")
    x = case_input(name)
    codes, lut, scale = oracle.uniform_8bit_quantize(x, "literal")
    assert oracle.norm_literal(x) == golden[f"{key}/norm"][0]
    assert np.array_equal(np.array([scale]), golden[f"{key}/scale"], equal_nan=True)
    assert np.array_equal(codes, golden[f"{key}/codes"])
    assert lut_rel_err(lut, golden[f"{key}/lut"].astype(np.float64), scale if np.isfinite(scale) and scale > 0 else 1.0) < 2e-5


def test_exact_and_literal_scale_agree_at_small_n(oracle):
    # up to 2^16 elements the fp32 accumulation error of libtorch's norm stays under 1e-6
    for name in CASES[:6]:
        x = case_input(name)
        if x.size < 2:
            continue
        a, b = float(oracle.scale_exact(x)), float(oracle.scale_literal(x))
        assert abs(a - b) <= 1e-6 * abs(b)


# ---------------------------------------------------------------- index add / set (collectives.cpp:8-22)

def test_index_add_and_set_are_numpy_gathers(oracle):
    rng = np.random.default_rng(9)
    lut = rng.standard_normal(256).astype(np.float32)
    codes = rng.integers(0, 256, 100003).astype(np.uint8)
    base = rng.standard_normal(100003).astype(np.float32)
    for threads in (1, 8):
        out = base.copy()
        oracle.index_add(out, lut, codes, threads)
        assert np.array_equal(out, base + lut[codes])
        oracle.index_set(out, lut, codes, threads)
        assert np.array_equal(out, lut[codes])


def test_div_scalar_is_libtorch_div(oracle):
    import torch

    y = np.random.default_rng(4).standard_normal(1000).astype(np.float32)
    for d in (2.0, 3.0, 8.0):
        z = y.copy()
        oracle.div_scalar(z, d)
        assert np.array_equal(z, torch.from_numpy(y.copy()).div_(d).numpy())


# ---------------------------------------------------------------- ring schedule (collectives.cpp:76-230)

def test_chunk_bounds_match_torch_chunk(oracle):
    import torch

    for n, parts in [(16, 4), (17, 4), (5, 8), (1, 4), (1000000, 16), (10, 3)]:
        got = oracle.torch_chunk_bounds(n, parts)
        want = [c.numel() for c in torch.arange(n).chunk(parts)]
        assert [hi - lo for lo, hi in got] == want


@pytest.mark.parametrize("W", [1, 2, 4])
def test_ring_sim_all_ranks_agree_on_owner_chunks_and_error_is_bounded(oracle, W):
    n = 2 * W * 4096
    rng = np.random.default_rng(W)
    xs = [(rng.standard_normal(n) * 10).astype(np.float32) for _ in range(W)]
    exact = np.sum(np.stack(xs).astype(np.float64), axis=0)
    ts = [x.copy() for x in xs]
    oracle.ring_allreduce_sim(ts, avg=False)
    err = [np.linalg.norm(t - exact) / math.sqrt(n) for t in ts]
    # the reference's own acceptance bound is 0.5 on the difference of two such errors
    # (tests/test_c/test_collectives.py:57); the error itself is a fraction of one bin width,
    # and a bin is 6 sigma / 256 of a sum with sigma = 10 sqrt(W)
    bin_width = 6 * 10 * math.sqrt(W) / 256
    assert max(err) < 1.5 * bin_width * math.sqrt(max(W - 1, 1))
    # rank r's own chunks are what everybody else ends up with after phase 2, up to the
    # requantization of already-quantized data on the way (collectives.cpp:215)
    for t in ts[1:]:
        assert np.linalg.norm(t - ts[0]) / math.sqrt(n) < bin_width


def test_ring_sim_avg_divides_by_world_size(oracle):
    W, n = 2, 2 * 2 * 2048
    rng = np.random.default_rng(8)
    xs = [(rng.standard_normal(n)).astype(np.float32) for _ in range(W)]
    ts = [x.copy() for x in xs]
    oracle.ring_allreduce_sim(ts, avg=True)
    exact = np.mean(np.stack(xs).astype(np.float64), axis=0)
    assert np.linalg.norm(ts[0] - exact) / math.sqrt(n) < 6 / 256


def test_ring_hops_accumulate(oracle):
    rng = np.random.default_rng(12)
    chunks = [(rng.standard_normal(8192) * 1e-3).astype(np.float32) for _ in range(4)]
    sent, acc = oracle.ring_hops(chunks)
    assert len(sent) == 4
    exact = np.sum(np.stack(chunks).astype(np.float64), axis=0)
    total_scale = sum(float(s[2]) for s in sent[:-1])
    inside = np.ones(8192, bool)
    for codes, _, _ in sent[:-1]:
        inside &= (codes > 0) & (codes < 255)
    assert np.abs(acc[inside] - exact[inside]).max() <= total_scale


# ---------------------------------------------------------------- the compiled reference, when built

def test_oracle_against_compiled_reference(oracle):
    if not oracle.ref_available():
        pytest.skip("oracle/_ref not built (the reference checkout is not present)")
    import torch
    from tests.conftest import lut_rel_err

    R = oracle.ref()
    rng = np.random.default_rng(21)
    for n in (3, 1000, 65543, (1 << 21) + 3):
        x = (rng.standard_t(3, n) * 1e-4).astype(np.float32)
        rc, rl = R.uniform_8bit_quantize(torch.from_numpy(x.copy()), True)
        oc, ol, sc = oracle.uniform_8bit_quantize(x, "literal")
        assert np.array_equal(rc.numpy(), oc)
        assert lut_rel_err(ol, rl.numpy().astype(np.float64), sc) < 5e-5
        q = R.quantize_per_tensor_uint8(torch.from_numpy(x.copy()), 3e-5, 100).numpy()
        assert np.array_equal(q, oracle.quantize_per_tensor_uint8(x, 3e-5, 100))


def special_tensors(n, rng):
    """Tensors that leave the ordinary branch of compression.cpp:113-122: a not-a-number (the norm, the
    scale and every product are NaN: all codes 0), an infinity (infinite scale, 1 / scale = 0: every
    finite element gets code 128, the infinity NaN -> code 0), values whose squares overflow fp32 but
    not fp64 (an ordinary tensor for an fp64 sum of squares), and values whose norm overflows fp32
    (infinite scale again)."""
    base = (rng.standard_normal(n) * 1e-3 + 5e-3).astype(np.float32)
    nan = base.copy()
    nan[n // 3] = np.nan
    inf = base.copy()
    inf[2 * n // 3] = np.inf
    big = (rng.standard_normal(n) * 1e25).astype(np.float32)
    huge = np.full(n, 3e38, np.float32)
    huge[::2] = np.float32(-2.5e38)
    return {"one NaN": nan, "one +inf": inf, "squares overflow fp32": big, "norm overflows fp32": huge}


def test_oracle_against_compiled_reference_on_special_values(oracle):
    # the branches a NaN, an infinity and an overflowing norm take: codes and scale of the restatement against
    # the reference's own compression.cpp, the table where the reference's fp32 sums are exact or infinite
    if not oracle.ref_available():
        pytest.skip("oracle/_ref not built (the reference checkout is not present)")
    import torch

    R = oracle.ref()
    rng = np.random.default_rng(22)
    for n in (1000, 65543):
        for label, x in special_tensors(n, rng).items():
            rc, rl = R.uniform_8bit_quantize(torch.from_numpy(x.copy()), True)
            if label == "squares overflow fp32":
                # libtorch's fp32 norm overflows where the formula's value is finite: the reference's scale is
                # infinite, the exact one is not (a reference artefact, like its drift at large n)
                oc, ol, sc = oracle.uniform_8bit_quantize(x, "literal")
                assert np.isinf(sc) and np.isfinite(oracle.scale_exact(x))
            else:
                oc, ol, sc = oracle.uniform_8bit_quantize(x, "exact")
                assert np.array_equal(np.array([sc]), np.array([oracle.scale_literal(x)]), equal_nan=True), label
            assert np.array_equal(rc.numpy(), oc), label
            assert np.array_equal(np.isnan(rl.numpy()), np.isnan(ol)), label
            assert np.array_equal(np.isinf(rl.numpy()), np.isinf(ol)), label
            if label == "one NaN":
                assert not oc.any() and np.isnan(ol[0]) and not ol[1:].any()
            if label == "one +inf":
                assert (oc == 128).sum() == n - 1 and oc[2 * n // 3] == 0 and np.isposinf(ol[0])


# ---------------------------------------------------------------- callers of the path (src/zeroband/diloco.py)

def test_pseudo_gradient_is_torch_sub_then_div(oracle):
    import torch

    rng = np.random.default_rng(13)
    for n in (1, 7, 1000, 65543):
        a = rng.standard_normal(n).astype(np.float32)
        b = (a + rng.standard_normal(n).astype(np.float32) * 1e-3).astype(np.float32)
        for W in (1.0, 2.0, 3.0, 8.0, 14.0):
            want = (torch.from_numpy(a) - torch.from_numpy(b)).div_(W).numpy()       # diloco.py:96-101
            assert np.array_equal(oracle.pseudo_gradient(a, b, W), want)


def test_outer_sgd_nesterov_is_torch_sgd_bit_for_bit(oracle):
    # the reference's outer optimizer: torch.optim.SGD(lr=outer_lr, momentum=0.9, nesterov=True) (diloco.py:72-74)
    import torch

    rng = np.random.default_rng(14)
    for n in (1, 3, 8, 15, 17, 33, 1003, 65541):
        for lr, mu in ((0.7, 0.9), (0.1, 0.5), (1.0, 0.9)):
            p0 = rng.standard_normal(n).astype(np.float32)
            p = torch.nn.Parameter(torch.from_numpy(p0.copy()))
            opt = torch.optim.SGD([p], lr=lr, momentum=mu, nesterov=True)
            mine = p0.copy()
            buf = np.zeros(n, np.float32)
            for step in range(3):
                g = (rng.standard_normal(n) * 1e-2).astype(np.float32)
                p.grad = torch.from_numpy(g.copy())
                opt.step()
                oracle.outer_sgd_nesterov(mine, buf, g, lr, mu, first_step=(step == 0))
                assert np.array_equal(mine, p.detach().numpy()), (n, lr, mu, step)
                assert np.array_equal(buf, opt.state[p]["momentum_buffer"].numpy()), (n, lr, mu, step)


@pytest.mark.parametrize("name", ["normal:1048583", "student:4194304", "normal:16777216", "normal:67108864", "normal:268435456"])
def test_oracle_reproduces_the_large_digests_of_the_compiled_reference(oracle, name):
    # sizes where libtorch's norm visibly differs from the exact one: the literal restatement must give
    # the reference's scale bits and codes (SHA-256 and populations written by tests/golden/make_fixtures.py)
    import hashlib
    import json
    from pathlib import Path

    from tests.golden.make_fixtures import case_input

    want = json.loads((Path(__file__).parent / "golden" / "uniform8_reference_large.json").read_text())[name]
    x = case_input(name)
    assert hashlib.sha256(x.tobytes()).hexdigest() == want["input_sha256"]      # the generator still draws the same input
    assert int(np.array([oracle.norm_literal(x)], np.float32).view(np.uint32)[0]) == want["norm_bits"]
    codes, lut, scale = oracle.uniform_8bit_quantize(x, "literal")
    assert int(np.array([scale], np.float32).view(np.uint32)[0]) == want["scale_bits"]
    assert hashlib.sha256(codes.tobytes()).hexdigest() == want["codes_sha256"]
    assert np.bincount(codes, minlength=256).tolist() == want["counts"]
    ref_lut = np.array(want["lut"], np.float32)
    assert np.abs(lut - ref_lut).max() <= 2e-5 * max(1.0, 2.0 * x.size / (1 << 24)) * max(float(scale), np.abs(ref_lut).max())
    # and the exact scale is larger, by libtorch's accumulation loss (-7e-4 at 2^24, -5e-3 at 2^26, -3.7e-2 at 2^28)
    rel = float(scale) / float(oracle.scale_exact(x)) - 1
    assert -5e-2 < rel <= 0
    if x.size >= 1 << 26:
        assert rel < -2e-3


def closed_form_ring_inputs(W: int, csz: int):
    """Rank r's chunk c is the constant 100 (r + 1) + c, except that chunk 1 sums to zero over the
    ranks and chunk 0 is negative.  A constant chunk quantizes without loss (every element in one
    bin whose mean is the constant; an all-zero chunk in code 0 with mean 0), and every partial sum
    is a small integer, so ring_allreduce must return exactly sum_r v[r, c] in every element of
    chunk c on every rank: one misrouted, dropped or repeated message changes that."""
    import numpy as np

    nb = 2 * W
    v = np.zeros((W, nb), np.float32)
    for r in range(W):
        for c in range(nb):
            v[r, c] = 100 * (r + 1) + c
    v[:, 0] *= -1
    if W > 1:
        v[:, 1] = np.arange(W) - (W - 1) / 2.0 if W % 2 else np.arange(W) * 2 - (W - 1)      # sums to zero, integers
    tensors = [np.repeat(v[r], csz).astype(np.float32) for r in range(W)]
    return v, tensors


@pytest.mark.parametrize("W", [1, 2, 3, 4, 8])
@pytest.mark.parametrize("avg", [False, True])
def test_ring_sim_closed_form_on_chunkwise_constant_inputs(oracle, W, avg):
    # pins the chunk-index algebra (collectives.cpp:116, 192), the forwarding condition (:136, :212),
    # the division for AVG (:155-159) and the own-chunk round trip (:161-173) exactly
    csz = 512
    v, tensors = closed_form_ring_inputs(W, csz)
    oracle.ring_allreduce_sim(tensors, avg=avg)
    total = v.sum(axis=0, dtype=np.float64).astype(np.float32)
    want = total / np.float32(W) if avg else total
    for r in range(W):
        got = tensors[r].reshape(2 * W, csz)
        for c in range(2 * W):
            assert np.all(got[c] == want[c]), (W, avg, r, c, got[c][:3], want[c])
