"""Full-size runs (2^28 elements; 2^26-element ring chunks) checked through properties that
do not need the CPU oracle: torch on the GPU is used as a plain calculator here."""
import numpy as np
import pytest
import torch

from prime_amd import _lib
from tests.conftest import tables_agree
from tests.gpu_util import Abi, announce

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def abi(dev):
    return Abi(dev)


def test_uniform_8bit_quantize_2p28_properties(abi):
    n = 1 << 28
    g = torch.Generator(device=abi.dev).manual_seed(0)
    x = torch.randn(n, device=abi.dev, generator=g) * 1e-3
    announce("2^28 uniform")
    codes, lut, qp = abi.uniform(x)
    torch.cuda.synchronize()
    q = abi.qparams(qp)
    # scale: the reference's formula on an fp64 sum of squares
    sumsq = float((x.double() ** 2).sum())
    want = np.float32(6.0 * (float(np.float32(np.sqrt(sumsq))) / np.sqrt(n - 1)) / 256.0)
    assert abs(q["sumsq"] - sumsq) <= 1e-12 * sumsq
    assert abs(float(q["scale"]) - float(want)) <= 1e-6 * float(want)
    assert abs(q["sum"] - float(x.double().sum())) <= 1e-12 * float(x.double().abs().sum())
    # codes: the same arithmetic spelled with torch ops (multiply, round half away, clamp)
    inv = torch.tensor(1.0, dtype=torch.float32) / torch.tensor(float(q["scale"]), dtype=torch.float32)
    p = x * float(inv)
    r = torch.where(p >= 0, torch.floor(p + 0.5), torch.ceil(p - 0.5))
    r = torch.where((p - torch.trunc(p)).abs() == 0.5, torch.trunc(p) + torch.sign(p), torch.round(p))
    want_codes = (r.clamp(-128, 127) + 128).to(torch.uint8)
    assert torch.equal(codes, want_codes)
    del p, r, want_codes
    # lookup: counts add up, count-weighted means give back the sum, bins are ordered
    cnt = torch.bincount(codes.view(-1).int(), minlength=256).double()
    assert int(cnt.sum()) == n
    sums = torch.bincount(codes.view(-1).int(), weights=x.double(), minlength=256)     # (index_add_ takes 40 s here)
    mean = torch.where(cnt > 0, sums / cnt.clamp(min=1), torch.zeros_like(sums))
    err = (lut.double() - mean).abs() / torch.maximum(mean.abs(), torch.tensor(float(q["scale"]), device=abi.dev, dtype=torch.float64))
    assert float(err.max()) <= 1e-6
    assert abs(float((cnt * lut.double()).sum()) - float(x.double().sum())) <= 1e-6 * float(x.double().abs().sum())
    filled = lut[cnt > 0]
    assert bool((filled[1:] > filled[:-1]).all())
    # dequantize: a gather, and within one bin width of the input for unclipped elements
    out = torch.empty_like(x)
    abi.dequant(out, lut, codes, add=False)
    assert torch.equal(out, lut[codes.long()])
    inside = (codes > 0) & (codes < 255)
    assert float((out - x)[inside].abs().max()) <= float(q["scale"])
    del out, inside
    # the default walk spreads the cached end of the tensor among the other tiles and keeps that end out of the
    # statistics pass's load hint: without either, the same codes, table and statistics record bit for bit
    saved = {k: _lib.get_option(k) for k in ("mix_cached", "stats_keep_mib")}
    try:
        for mix, keep in ((0, saved["stats_keep_mib"]), (0, 0)):
            _lib.set_option("mix_cached", mix)
            _lib.set_option("stats_keep_mib", keep)
            announce(f"2^28 uniform mix_cached={mix} stats_keep_mib={keep}")
            c2, l2, q2 = abi.uniform(x)
            torch.cuda.synchronize()
            assert torch.equal(c2, codes) and torch.equal(l2.view(torch.int32), lut.view(torch.int32))
            assert torch.equal(q2.view(torch.int64), qp.view(torch.int64))
    finally:
        for k, v in saved.items():
            _lib.set_option(k, v)


@pytest.mark.parametrize("n", [70_000_001, (1 << 27), (1 << 27) + 4096 * 3 + 5, 200_000_003])
def test_large_tensors_around_the_cache_thresholds(abi, n):
    # 267 MiB (the end kept, walked from the end), 512 MiB (exactly twice the kept size: the mixed walk begins), a ragged
    # size just above, 763 MiB with an odd element count: codes against the formula, counts, and the same call with the
    # cache-aware paths switched off bit for bit
    x = torch.randn(n, device=abi.dev, generator=torch.Generator(device=abi.dev).manual_seed(n % 1000)) * 1e-3
    x[n // 3] = 0.9                                         # beyond the fixed-point range: the fp64 side sums
    announce(f"large uniform n={n}")
    codes, lut, qp = abi.uniform(x)
    torch.cuda.synchronize()
    q = abi.qparams(qp)
    sumsq = float((x.double() ** 2).sum())
    assert abs(q["sumsq"] - sumsq) <= 1e-12 * sumsq
    inv = float(torch.tensor(1.0, dtype=torch.float32) / torch.tensor(float(q["scale"]), dtype=torch.float32))
    p = x * inv
    r = torch.where((p - torch.trunc(p)).abs() == 0.5, torch.trunc(p) + torch.sign(p), torch.round(p))
    assert torch.equal(codes, (r.clamp(-128, 127) + 128).to(torch.uint8))
    del p, r
    cnt = torch.bincount(codes.int(), minlength=256)
    assert int(cnt.sum()) == n
    sums = torch.bincount(codes.int(), weights=x.double(), minlength=256)
    mean = torch.where(cnt > 0, sums / cnt.clamp(min=1).double(), torch.zeros_like(sums))
    floor = torch.tensor(float(q["scale"]), device=abi.dev, dtype=torch.float64)
    assert float(((lut.double() - mean).abs() / torch.maximum(mean.abs(), floor)).max()) <= 1e-6
    saved = {k: _lib.get_option(k) for k in ("mix_cached", "stats_keep_mib")}
    try:
        _lib.set_option("mix_cached", 0)
        _lib.set_option("stats_keep_mib", 0)
        announce(f"large uniform n={n}, plain walk")
        c2, l2, q2 = abi.uniform(x)
        torch.cuda.synchronize()
        assert torch.equal(c2, codes) and torch.equal(q2.view(torch.int64), qp.view(torch.int64))
        assert torch.equal(l2.view(torch.int32)[1:255], lut.view(torch.int32)[1:255])        # one far element, in entry 255
        assert torch.allclose(l2[[0, 255]], lut[[0, 255]], rtol=1e-6, atol=0)
    finally:
        for k, v in saved.items():
            _lib.set_option(k, v)


def test_ring_reduce_step_2p26_chunks(abi):
    # benchmark configuration 3 in full: W = 8 ranks' 2^26-element chunks N(0, 1e-3), seed = rank; chunk 0 is
    # quantized, then all 7 hops of dequantize-add + requantize, each checked through properties
    n = 1 << 26
    x0 = torch.randn(n, device=abi.dev, generator=torch.Generator(device=abi.dev).manual_seed(0)) * 1e-3
    announce("2^26 ring: quantize rank 0")
    codes, lut, _ = abi.uniform(x0)
    del x0
    for r in range(1, 8):
        acc = torch.randn(n, device=abi.dev, generator=torch.Generator(device=abi.dev).manual_seed(r)) * 1e-3
        want = acc + lut[codes.long()]
        announce(f"2^26 ring hop {r}")
        codes, lut, qp = abi.ring_step(acc, codes, lut)
        torch.cuda.synchronize()
        assert torch.equal(acc, want)
        q = abi.qparams(qp)
        sumsq = float((want.double() ** 2).sum())
        assert abs(q["sumsq"] - sumsq) <= 1e-12 * sumsq
        exact = np.float32(6.0 * (float(np.float32(np.sqrt(sumsq))) / np.sqrt(n - 1)) / 256.0)
        assert abs(float(q["scale"]) - float(exact)) <= 1e-6 * float(exact)
        cnt = torch.bincount(codes.int(), minlength=256)
        assert int(cnt.sum()) == n
        inside = (codes > 0) & (codes < 255)
        assert float((lut[codes.long()] - want)[inside].abs().max()) <= float(q["scale"])
        sums = torch.bincount(codes.int(), weights=want.double(), minlength=256)
        mean = torch.where(cnt > 0, sums / cnt.clamp(min=1).double(), torch.zeros_like(sums))
        floor = torch.tensor(float(q["scale"]), device=abi.dev, dtype=torch.float64)
        assert float(((lut.double() - mean).abs() / torch.maximum(mean.abs(), floor)).max()) <= 1e-6
        del want, acc


def test_ring_reduce_step_2p28_all_three_kinds(abi):
    # the ring steps at the size the second headline figure is quoted on (1 GiB accumulators: hinted loads in the
    # accumulate pass, four-row tiles and tiles on demand in the quantize pass that follows a writer): reduce,
    # reduce with the division of AVG, gather; accumulator bit for bit against torch, codes recomputed from the
    # derived scale, table against the bin means
    n = 1 << 28
    msg = torch.randn(n, device=abi.dev, generator=torch.Generator(device=abi.dev).manual_seed(40)) * 1e-3
    mc, ml, _ = abi.uniform(msg)
    del msg
    for kind, divisor in (("reduce", None), ("reduce_div", 8.0), ("gather", None)):
        acc = torch.randn(n, device=abi.dev, generator=torch.Generator(device=abi.dev).manual_seed(41)) * 1e-3
        if kind == "gather":
            want = ml[mc.long()]
        else:
            want = acc + ml[mc.long()]
            if divisor:
                want = want / divisor
        announce(f"2^28 ring step {kind}")
        codes, lut, qp = abi.ring_step(acc, mc, ml, gather=(kind == "gather"), divisor=divisor)
        torch.cuda.synchronize()
        assert torch.equal(acc.view(torch.int32), want.view(torch.int32))
        del acc
        q = abi.qparams(qp)
        sumsq = float((want.double() ** 2).sum())
        assert abs(q["sumsq"] - sumsq) <= 1e-12 * sumsq
        exact = np.float32(6.0 * (float(np.float32(np.sqrt(sumsq))) / np.sqrt(n - 1)) / 256.0)
        assert abs(float(q["scale"]) - float(exact)) <= 1e-6 * float(exact)
        inv = float(torch.tensor(1.0, dtype=torch.float32) / torch.tensor(float(q["scale"]), dtype=torch.float32))
        p = want * inv
        r = torch.where((p - torch.trunc(p)).abs() == 0.5, torch.trunc(p) + torch.sign(p), torch.round(p))
        assert torch.equal(codes, (r.clamp(-128, 127) + 128).to(torch.uint8))
        del p, r
        cnt = torch.bincount(codes.int(), minlength=256)
        assert int(cnt.sum()) == n
        sums = torch.bincount(codes.int(), weights=want.double(), minlength=256)
        mean = torch.where(cnt > 0, sums / cnt.clamp(min=1).double(), torch.zeros_like(sums))
        floor = torch.tensor(float(q["scale"]), device=abi.dev, dtype=torch.float64)
        assert float(((lut.double() - mean).abs() / torch.maximum(mean.abs(), floor)).max()) <= 1e-6
        del want, codes


def test_config2_all_22_layer_buckets(abi):
    # benchmark configuration 2 in full: 22 per-layer buckets of 51,380,224 elements, Student-t(3) * 1e-4
    # (heavy tails: the clip bins fill), quantized bucket by bucket; every bucket is checked on the
    # device through what holds at any size: the scale formula on the fp64 norm, codes recomputed
    # from that scale, bin populations, the table against fp64 bin means, the round trip
    n, layers = 4 * 2048 * 2048 + 3 * 2048 * 5632, 22
    g = torch.Generator(device=abi.dev).manual_seed(2)
    for layer in range(layers):
        # Student-t(3) = normal / sqrt(chi2(3) / 3)
        z = torch.randn(n, device=abi.dev, generator=g)
        chi = (torch.randn(3, n, device=abi.dev, generator=g) ** 2).sum(0)
        x = (z / torch.sqrt(chi / 3.0) * 1e-4).float()
        del z, chi
        if layer % 4 == 0:
            announce(f"cfg2 layer {layer}")
        codes, lut, qp = abi.uniform(x)
        q = abi.qparams(qp)
        sumsq = float((x.double() ** 2).sum())
        want = np.float32(6.0 * (float(np.float32(np.sqrt(sumsq))) / np.sqrt(n - 1)) / 256.0)
        assert abs(float(q["scale"]) - float(want)) <= 1e-6 * float(want), layer
        # codes from the scale the kernel derived: round half away from zero, +128, clamp (compression.cpp:23-24)
        p = x * (torch.tensor(1.0, device=abi.dev) / torch.tensor(float(q["scale"]), device=abi.dev))
        whole = torch.trunc(p)                                     # p - whole is exact: no p + 0.5 that could round up
        rounded = whole + ((p - whole).abs() >= 0.5) * torch.sign(p)
        ref_codes = (rounded + 128).clamp(0, 255).to(torch.uint8)
        del whole, rounded
        assert torch.equal(codes, ref_codes), (layer, int((codes != ref_codes).sum()))
        cnt = torch.bincount(codes.int(), minlength=256)
        assert int(cnt.sum()) == n
        assert int(cnt[0]) > n // 1000 and int(cnt[255]) > n // 1000      # the tails clip
        sums = torch.bincount(codes.int(), weights=x.double(), minlength=256)
        mean = torch.where(cnt > 0, sums / cnt.clamp(min=1), torch.zeros_like(sums))
        floor = torch.tensor(float(q["scale"]), device=abi.dev, dtype=torch.float64)
        assert float(((lut.double() - mean).abs() / torch.maximum(mean.abs(), floor)).max()) <= 1e-6, layer
        out = torch.empty_like(x)
        abi.dequant(out, lut, codes, add=False)
        assert torch.equal(out, lut[codes.long()]), layer
        inside = (codes > 0) & (codes < 255)
        assert float((out - x)[inside].abs().max()) <= float(q["scale"]), layer
        del x, p, ref_codes, out, inside


def test_config4_shard_all_42_buckets(abi):
    # benchmark configuration 4 in full: 1.25e9 elements (5 GB) as 42 buckets, the last 32 longer, N(0, 5e-4)
    # with 0.01 % of entries at +-50 sigma; quantize + lookup + dequantize per bucket, checked through
    # properties that hold at any size
    base, extra, nb = 29_761_904, 32, 42
    assert base * nb + extra == 1_250_000_000
    g = torch.Generator(device=abi.dev).manual_seed(4)
    sigma = 5e-4
    for b in range(nb):
        n = base + (extra if b == nb - 1 else 0)
        x = torch.randn(n, device=abi.dev, generator=g) * sigma
        k = n // 10000
        pos = torch.randint(0, n, (k,), device=abi.dev, generator=g)
        sign = torch.where(torch.rand(k, device=abi.dev, generator=g) < 0.5, -1.0, 1.0)
        x[pos] = sign * (50 * sigma)
        if b % 6 == 0:
            announce(f"cfg4 bucket {b}")
        codes, lut, qp = abi.uniform(x)
        out = torch.empty_like(x)
        abi.dequant(out, lut, codes, add=False)
        if b % 6 and b != nb - 1:
            continue                      # every bucket runs; a sample of them is checked in full
        q = abi.qparams(qp)
        sumsq = float((x.double() ** 2).sum())
        want = np.float32(6.0 * (float(np.float32(np.sqrt(sumsq))) / np.sqrt(n - 1)) / 256.0)
        assert abs(float(q["scale"]) - float(want)) <= 1e-6 * float(want)
        cnt = torch.bincount(codes.int(), minlength=256)
        assert int(cnt.sum()) == n
        c = codes[pos]
        assert bool(((c == 0) | (c == 255)).all())                    # outliers clip
        assert torch.equal(out, lut[codes.long()])
        inside = (codes > 0) & (codes < 255)
        assert float((out - x)[inside].abs().max()) <= float(q["scale"])
        sums = torch.bincount(codes.view(-1).int(), weights=x.double(), minlength=256)
        mean = torch.where(cnt > 0, sums / cnt.clamp(min=1), torch.zeros_like(sums))
        floor = torch.tensor(float(q["scale"]), device=abi.dev, dtype=torch.float64)
        assert float(((lut.double() - mean).abs() / torch.maximum(mean.abs(), floor)).max()) <= 1e-6


def test_all_gather_requantization_2p26_chunk_in_the_code_domain(abi):
    # config 3's chunk: what the all-gather forwards, from codes alone, against the fp32 route
    n = 1 << 26
    g = torch.Generator(device=abi.dev).manual_seed(5)
    src = torch.randn(n, device=abi.dev, generator=g) * 1e-3
    announce("2^26 requantize codes")
    codes_in, lut_in, _ = abi.uniform(src)
    codes, lut, qp = abi.requantize_codes(codes_in, lut_in)
    chunk = torch.empty(n, device=abi.dev)
    codes2, lut2, qp2 = abi.ring_step(chunk, codes_in, lut_in, gather=True)
    torch.cuda.synchronize()
    assert torch.equal(chunk, lut_in[codes_in.long()])
    assert torch.equal(codes, codes2)
    q, q2 = abi.qparams(qp), abi.qparams(qp2)
    assert q["scale"] == q2["scale"] and q["n"] == n
    assert abs(q["sumsq"] - q2["sumsq"]) <= 1e-12 * q2["sumsq"]
    assert tables_agree(lut.cpu().numpy(), lut2.cpu().numpy(), q["scale"], 2e-6)
    # exact population-weighted means, spelled with torch
    cnt = torch.bincount(codes_in.int(), minlength=256).double()
    new = torch.zeros(256, dtype=torch.float64, device=abi.dev)
    pop = torch.zeros(256, dtype=torch.float64, device=abi.dev)
    mapping = torch.zeros(256, dtype=torch.long, device=abi.dev)
    mapping[codes_in.long()] = codes.long()               # a function of the old code
    assert torch.equal(mapping[codes_in.long()], codes.long())
    new.index_add_(0, mapping, cnt * lut_in.double())
    pop.index_add_(0, mapping, cnt)
    want = torch.where(pop > 0, new / pop.clamp(min=1), torch.zeros_like(new)).float()
    assert tables_agree(lut.cpu().numpy(), want.cpu().numpy(), q["scale"], 1e-6)


def test_ring_first_touch_2p26_chunk_equals_separate_calls(abi):
    from prime_amd import _lib

    n = 1 << 26
    g = torch.Generator(device=abi.dev).manual_seed(6)
    outer = torch.randn(n, device=abi.dev, generator=g)
    inner = outer + torch.randn(n, device=abi.dev, generator=g) * 1e-3
    msg_c, msg_l, _ = abi.uniform(torch.randn(n, device=abi.dev, generator=g) * 1e-4)
    for with_msg, divisor in ((False, 1.0), (True, 1.0), (True, 8.0)):
        announce(f"2^26 first touch msg={with_msg} divisor={divisor}")
        grad = torch.empty(n, device=abi.dev)
        codes = torch.empty(n, dtype=torch.uint8, device=abi.dev)
        lut = torch.empty(256, device=abi.dev)
        qp = torch.empty(4, dtype=torch.float64, device=abi.dev)
        _lib.check(abi.lib.prime_ring_first_touch(outer.data_ptr(), inner.data_ptr(), n, 8.0,
                                                  msg_c.data_ptr() if with_msg else None, msg_l.data_ptr() if with_msg else None,
                                                  divisor, grad.data_ptr(), codes.data_ptr(), lut.data_ptr(), qp.data_ptr(),
                                                  abi.ws.data_ptr(), abi.st), "first touch")
        want = (outer - inner) / 8.0
        if with_msg:
            want = want + msg_l[msg_c.long()]
            if divisor != 1.0:
                want = want / divisor
        codes2, lut2, qp2 = abi.uniform(want)
        torch.cuda.synchronize()
        assert torch.equal(grad, want)
        assert torch.equal(codes, codes2)
        assert abi.qparams(qp)["scale"] == abi.qparams(qp2)["scale"]
        assert tables_agree(lut.cpu().numpy(), lut2.cpu().numpy(), abi.qparams(qp)["scale"], 2e-6)


def test_more_than_2p31_elements_in_one_call(abi):
    # indices past 32 bits: 2^31 + 4099 elements (8.6 GB) through quantize, requantize-from-codes and
    # dequantize; checked piecewise with torch as the calculator
    n = (1 << 31) + 4099
    piece = 1 << 27
    x = torch.empty(n, device=abi.dev)
    g = torch.Generator(device=abi.dev).manual_seed(31)
    for lo in range(0, n, piece):
        x[lo:lo + piece].normal_(generator=g).mul_(1e-3)
    x[-1] = 0.05                                           # a clipped element at the very end
    announce("2^31+4099 uniform")
    codes, lut, qp = abi.uniform(x)
    torch.cuda.synchronize()
    q = abi.qparams(qp)
    assert q["n"] == n
    sumsq = sum(float((x[lo:lo + piece].double() ** 2).sum()) for lo in range(0, n, piece))
    assert abs(q["sumsq"] - sumsq) <= 1e-12 * sumsq
    want_scale = np.float32(6.0 * (float(np.float32(np.sqrt(sumsq))) / np.sqrt(n - 1)) / 256.0)
    assert abs(float(q["scale"]) - float(want_scale)) <= 1e-6 * float(want_scale)
    inv = float(torch.tensor(1.0, dtype=torch.float32) / torch.tensor(float(q["scale"]), dtype=torch.float32))
    cnt = torch.zeros(256, dtype=torch.int64, device=abi.dev)
    sums = torch.zeros(256, dtype=torch.float64, device=abi.dev)
    for lo in range(0, n, piece):
        xs, cs = x[lo:lo + piece], codes[lo:lo + piece]
        p = xs * inv
        r = torch.where((p - torch.trunc(p)).abs() == 0.5, torch.trunc(p) + torch.sign(p), torch.round(p))
        assert torch.equal(cs, (r.clamp(-128, 127) + 128).to(torch.uint8)), lo
        ci = cs.int()
        cnt += torch.bincount(ci, minlength=256)
        sums += torch.bincount(ci, weights=xs.double(), minlength=256)     # per-workgroup histograms, no contended atomics
        del p, r, ci
        announce(f"2^31+4099 checked up to {lo + piece}")
    assert int(cnt.sum()) == n and int(codes[-1]) == 255
    mean = torch.where(cnt > 0, sums / cnt.clamp(min=1).double(), torch.zeros_like(sums))
    err = (lut.double() - mean).abs() / torch.maximum(mean.abs(), torch.tensor(float(q["scale"]), device=abi.dev, dtype=torch.float64))
    assert float(err.max()) <= 1e-6
    announce("2^31+4099 requantize codes")
    codes2, lut2, qp2 = abi.requantize_codes(codes, lut)
    torch.cuda.synchronize()
    q2 = abi.qparams(qp2)
    want_sq = float((cnt.double() * lut.double() ** 2).sum())
    assert q2["n"] == n and abs(q2["sumsq"] - want_sq) <= 1e-12 * want_sq
    mapping = torch.zeros(256, dtype=torch.long, device=abi.dev)
    inv2 = float(torch.tensor(1.0, dtype=torch.float32) / torch.tensor(float(q2["scale"]), dtype=torch.float32))
    p = lut * inv2
    r = torch.where((p - torch.trunc(p)).abs() == 0.5, torch.trunc(p) + torch.sign(p), torch.round(p))
    mapping = (r.clamp(-128, 127) + 128).long()
    for lo in range(0, n, piece):
        assert torch.equal(codes2[lo:lo + piece].long(), mapping[codes[lo:lo + piece].long()]), lo
    announce("2^31+4099 dequantize")
    abi.dequant(x, lut, codes, add=False)                  # x is overwritten
    torch.cuda.synchronize()
    for lo in range(0, n, piece):
        assert torch.equal(x[lo:lo + piece], lut[codes[lo:lo + piece].long()]), lo
