"""Host-side mirror of the reference interface: names, signatures, error behaviour (CPU only)."""
import inspect
from pathlib import Path

import pytest
import torch
import torch.distributed as dist


def test_compression_enum_values():
    # src/zeroband/config.py:10-12
    from prime_amd.config import Compression

    assert Compression.NO.value == "no" and Compression.UINT8.value == "uint8"
    assert Compression("uint8") is Compression.UINT8


def test_python_signatures_match_the_reference_wrappers():
    # src/zeroband/C/compression.py:11,22,34 and src/zeroband/C/collectives.py:23-27, collectives.py:31-36
    from prime_amd.C import collectives as Cc
    from prime_amd.C import compression as C
    from prime_amd import collectives

    assert str(inspect.signature(C.uniform_8bit_quantize)) == \
        "(tensor: torch.Tensor, inplace: bool = True) -> Tuple[torch.Tensor, torch.Tensor]"
    assert list(inspect.signature(C.average_buckets).parameters) == ["tensor", "quant_weight", "n_bins"]
    assert list(inspect.signature(C.quantize_per_tensor_uint8).parameters) == ["tensor", "scale", "zero_point"]
    p = inspect.signature(Cc.ring_allreduce).parameters
    assert list(p) == ["tensor", "op", "group"] and p["op"].default == dist.ReduceOp.SUM and p["group"].default is None
    p = inspect.signature(collectives.all_reduce).parameters
    assert list(p) == ["compression", "tensor", "op", "group"]


def test_op_schemas():
    import prime_amd.ops  # noqa: F401

    want = {
        "uniform_8bit_quantize": "prime::uniform_8bit_quantize(Tensor tensor, bool inplace=True) -> (Tensor, Tensor)",
        "average_buckets": "prime::average_buckets(Tensor tensor, Tensor quant_weight, int n_bins) -> Tensor",
        "quantize_per_tensor_uint8": "prime::quantize_per_tensor_uint8(Tensor tensor, float scale, int zero_point) -> Tensor",
        "dequantize": "prime::dequantize(Tensor codes, Tensor lut) -> Tensor",
        "ring_reduce_step": "prime::ring_reduce_step(Tensor(a!) acc, Tensor codes_in, Tensor lut_in) -> (Tensor, Tensor)",
    }
    for name, schema in want.items():
        assert str(getattr(torch.ops.prime, name).default._schema) == schema


def test_cpu_tensors_reach_no_kernel():
    # the product has no CPU path: the dispatcher must refuse, not fall back
    from prime_amd.C import compression as C

    with pytest.raises(NotImplementedError):
        C.uniform_8bit_quantize(torch.randn(16))
    with pytest.raises(NotImplementedError):
        C.quantize_per_tensor_uint8(torch.randn(16), 0.1, 128)
    with pytest.raises(NotImplementedError):
        C.average_buckets(torch.randn(16), torch.zeros(16, dtype=torch.uint8), 256)


def test_fake_tensors_give_shapes():
    from torch._subclasses.fake_tensor import FakeTensorMode
    import prime_amd.ops  # noqa: F401

    with FakeTensorMode():
        x = torch.empty(3, 5)
        codes, lut = torch.ops.prime.uniform_8bit_quantize(x)
        assert codes.shape == (3, 5) and codes.dtype == torch.uint8 and lut.shape == (256,) and lut.dtype == torch.float32


def test_every_prime_op_traces_on_fake_tensors():
    # every op of the library has a shape-only implementation: a traced program can carry any of them
    from torch._subclasses.fake_tensor import FakeTensorMode
    import prime_amd.ops  # noqa: F401

    P = torch.ops.prime
    with FakeTensorMode():
        x = torch.empty(3, 5)
        flat = torch.empty(40)
        codes = torch.empty(40, dtype=torch.uint8)
        lut = torch.empty(256)
        u8 = (torch.uint8, torch.float32)

        def pair(out, shape):
            assert out[0].shape == shape and (out[0].dtype, out[1].dtype) == u8 and out[1].shape == (256,)

        calls = {
            "uniform_8bit_quantize": lambda: pair(P.uniform_8bit_quantize(x), (3, 5)),
            "uniform_8bit_quantize_literal": lambda: pair(P.uniform_8bit_quantize_literal(x), (3, 5)),
            "average_buckets": lambda: P.average_buckets(flat, codes, 300).shape == (300,) or pytest.fail("shape"),
            "quantize_per_tensor_uint8": lambda: P.quantize_per_tensor_uint8(x, 0.1, 128).dtype == torch.uint8 or pytest.fail("dtype"),
            "dequantize": lambda: P.dequantize(codes, lut).dtype == torch.float32 or pytest.fail("dtype"),
            "dequantize_": lambda: P.dequantize_(flat, codes, lut, True),
            "ring_reduce_step": lambda: pair(P.ring_reduce_step(flat, codes, lut), (40,)),
            "ring_gather_step": lambda: pair(P.ring_gather_step(flat, codes, lut), (40,)),
            "ring_reduce_div_step": lambda: pair(P.ring_reduce_div_step(flat, codes, lut, 4.0), (40,)),
            "requantize_codes": lambda: pair(P.requantize_codes(codes, lut), (40,)),
            "uniform_8bit_quantize_stats": lambda: P.uniform_8bit_quantize_stats(x)[2].shape == (4,) or pytest.fail("qparams"),
            "uniform_8bit_quantize_batched": lambda: P.uniform_8bit_quantize_batched(flat, torch.empty(6, dtype=torch.int64))[1].shape == (5, 256)
                                                     or pytest.fail("luts"),
            "div_": lambda: P.div_(flat, 2.0),
            "pseudo_gradient_": lambda: P.pseudo_gradient_(flat, flat.clone(), flat.clone(), 4.0),
            "ring_first_touch_": lambda: (pair(P.ring_first_touch_(flat, flat.clone(), flat.clone(), 4.0, codes, lut, 1.0), (40,)),
                                          pair(P.ring_first_touch_(flat, flat.clone(), flat.clone(), 4.0, None, None, 1.0), (40,))),
            "outer_sgd_nesterov_": lambda: (P.outer_sgd_nesterov_(flat, flat.clone(), flat.clone(), flat.clone(), 0.7, 0.9, True),
                                            P.outer_sgd_nesterov_(flat, flat.clone(), flat.clone(), None, 0.7, 0.9, False)),
            "outer_sgd_nesterov_codes_": lambda: P.outer_sgd_nesterov_codes_(flat, flat.clone(), codes, lut, flat.clone(), 0.7, 0.9, False),
        }
        for name, call in calls.items():
            call()
    defined = {s.name.split("::")[1] for s in torch._C._jit_get_all_schemas() if s.name.startswith("prime::")}
    assert defined == set(calls), defined ^ set(calls)


def test_ring_allreduce_rejects_other_reduce_ops():
    # collectives.cpp:83
    from prime_amd.C.collectives import ring_allreduce

    with pytest.raises(RuntimeError, match="Only SUM and AVG"):
        ring_allreduce(torch.zeros(8), dist.ReduceOp.MAX, None)


def test_fake_process_group_is_a_no_op():
    # src/zeroband/C/collectives.py:32-33
    from torch.testing._internal.distributed.fake_pg import FakeProcessGroup
    from prime_amd.collectives import Compression, all_reduce

    pg = FakeProcessGroup.__new__(FakeProcessGroup)
    x = torch.arange(8, dtype=torch.float32)
    all_reduce(Compression.UINT8, x, dist.ReduceOp.SUM, pg)
    assert torch.equal(x, torch.arange(8, dtype=torch.float32))


def test_simulated_ring_input_checks():
    from prime_amd.C.collectives import SimulatedRing, ring_allreduce

    a, b = torch.zeros(9), torch.zeros(9)
    with pytest.raises(ValueError, match="split into 4 chunks"):
        ring_allreduce(a, dist.ReduceOp.SUM, SimulatedRing([a, b]))      # torch.chunk(4) of 9 elements gives 3 pieces
    with pytest.raises(ValueError, match="not one of"):
        ring_allreduce(torch.zeros(8), dist.ReduceOp.SUM, SimulatedRing([torch.zeros(8), torch.zeros(8)]))
    d = a.double()
    with pytest.raises(RuntimeError, match="Float"):
        ring_allreduce(d, dist.ReduceOp.SUM, SimulatedRing([d]))


def test_missing_library_is_an_error(monkeypatch, tmp_path):
    from prime_amd import _lib

    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", tmp_path / "libprime_hip.so")
    with pytest.raises(_lib.PrimeHipError, match="no CPU fallback"):
        _lib.load()


def test_shim_registers_the_reference_import_paths():
    # src/zeroband/diloco.py:6, tests/test_c/test_compression.py:6: those imports, unchanged, reach this package
    import sys

    import prime_amd.shim as shim

    had = {k: sys.modules.get(k) for k in list(sys.modules) if k == "zeroband" or k.startswith("zeroband.")}
    try:
        shim.install()
        from zeroband.C.compression import average_buckets, quantize_per_tensor_uint8, uniform_8bit_quantize
        from zeroband.C.collectives import ring_allreduce
        from zeroband.collectives import Compression, all_reduce

        import prime_amd.C.collectives
        import prime_amd.C.compression
        import prime_amd.collectives

        assert uniform_8bit_quantize is prime_amd.C.compression.uniform_8bit_quantize
        assert average_buckets is prime_amd.C.compression.average_buckets
        assert quantize_per_tensor_uint8 is prime_amd.C.compression.quantize_per_tensor_uint8
        assert ring_allreduce is prime_amd.C.collectives.ring_allreduce
        assert all_reduce is prime_amd.collectives.all_reduce and Compression.UINT8.value == "uint8"
        shim.install()                                  # idempotent
        import zeroband.C.compression as again

        assert again is prime_amd.C.compression
    finally:
        shim.uninstall()
        for k in [k for k in sys.modules if k == "zeroband" or k.startswith("zeroband.")]:
            del sys.modules[k]
        sys.modules.update({k: v for k, v in had.items() if v is not None})


def test_bench_refuses_more_than_one_gpu():
    # one GPU per box: the benchmark says so instead of pretending to scale
    import subprocess
    import sys
    from pathlib import Path

    root = Path(__file__).resolve().parents[1]
    res = subprocess.run([sys.executable, str(root / "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert res.returncode == 2 and "one GPU" in res.stderr and res.stdout.strip() == ""


def test_short_rounding_sequence_equals_roundf_on_every_float_in_its_range(tmp_path):
    # the fused quantize pass rounds products within its fixed-point range with
    # trunc(c + copysign(0.49999997, c)); every one of the 2.3e9 floats of that range, on the host
    import subprocess

    src = Path(__file__).resolve().parent / "native" / "round_centre_check.c"
    exe = tmp_path / "round_centre_check"
    subprocess.run(["gcc", "-O2", "-ffp-contract=off", str(src), "-o", str(exe), "-lm"], check=True)
    res = subprocess.run([str(exe)], capture_output=True, text=True)
    assert res.returncode == 0, res.stdout
    assert "checked 2285502466 mismatches 0" in res.stdout


def _run_ranks(args, world, timeout=150):
    """One child process per rank of `python -m prime_amd.all_reduce_bench`, rendezvous on localhost."""
    import json
    import os
    import socket
    import subprocess
    import sys

    with socket.socket() as sock:
        sock.bind(("127.0.0.1", 0))
        port = sock.getsockname()[1]
    root = Path(__file__).resolve().parents[1]
    procs = []
    for r in range(world):
        env = dict(os.environ, PYTHONPATH=str(root), RANK=str(r), WORLD_SIZE=str(world), MASTER_ADDR="127.0.0.1",
                   MASTER_PORT=str(port), GLOO_SOCKET_IFNAME="lo")
        procs.append(subprocess.Popen([sys.executable, "-u", "-m", "prime_amd.all_reduce_bench", *args], cwd=str(root), env=env,
                                      stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True))
    outs = []
    try:
        for pr in procs:
            out, _ = pr.communicate(timeout=timeout)
            outs.append(out)
    finally:
        for pr in procs:
            if pr.poll() is None:
                pr.kill()
    for r, pr in enumerate(procs):
        assert pr.returncode == 0, f"rank {r} failed:\n{outs[r][-3000:]}"
    lines = [ln for ln in outs[0].splitlines() if ln.startswith("{")]
    assert len(lines) == 1, outs[0][-2000:]
    return json.loads(lines[0])


def test_all_reduce_timing_script_without_compression_on_two_host_ranks():
    # the reference's scripts/all_reduce.py with compression "no": the tensor stays on the host
    line = _run_ranks(["--size_model", "100001", "--n_iters", "2", "--compression", "no", "--check"], world=2)
    assert line["ranks"] == 2 and line["size_model"] == 100001 and line["compression"] == "no"
    assert line["MBps"] > 0 and line["rms_error"] < 1e-6


def _gloo_avg_worker(rank: int, world: int, port: int, q) -> None:
    import os

    os.environ.update(MASTER_ADDR="127.0.0.1", MASTER_PORT=str(port))
    dist.init_process_group("gloo", rank=rank, world_size=world)
    try:
        from prime_amd.collectives import gloo_all_reduce

        x = torch.arange(8, dtype=torch.float32) * (rank + 1)
        gloo_all_reduce(x, dist.ReduceOp.AVG)
        y = torch.ones(4) * (rank + 1)
        gloo_all_reduce(y, dist.ReduceOp.SUM)
        q.put((rank, x.tolist(), y.tolist()))
    finally:
        dist.destroy_process_group()


def test_uncompressed_all_reduce_averages_over_a_real_gloo_group():
    # src/zeroband/collectives.py:12-28 with op = AVG on host tensors: divide by the group size, then SUM
    # (Gloo has no AVG of its own); two ranks, CPU only
    import socket
    import torch.multiprocessing as mp

    with socket.socket() as s:
        s.bind(("127.0.0.1", 0))
        port = s.getsockname()[1]
    ctx = mp.get_context("spawn")
    q = ctx.Queue()
    procs = [ctx.Process(target=_gloo_avg_worker, args=(r, 2, port, q)) for r in range(2)]
    for p in procs:
        p.start()
    got = [q.get(timeout=120) for _ in procs]
    for p in procs:
        p.join(timeout=60)
        assert p.exitcode == 0
    for _, x, y in got:
        assert x == [1.5 * k for k in range(8)]       # (k + 2 k) / 2
        assert y == [3.0] * 4


def test_bench_takes_its_traffic_figure_from_the_committed_counter_summaries():
    # roofline.traffic is read from profiles/*_hbm_traffic.txt (the scaled FETCH_SIZE + WRITE_SIZE of the dominant
    # kernel), not typed into bench.py: the figure exists, belongs to that kernel and is the algorithmic 5 B per
    # element plus the histogram partials, with no wasted re-reads
    import re
    import sys
    from pathlib import Path

    root = Path(__file__).resolve().parents[1]
    sys.path.insert(0, str(root))
    import bench

    for profile, elems in (("uniform_2p28_hbm_traffic.txt", 1 << 28), ("cfg2_buckets_hbm_traffic.txt", bench.BUCKET_ELEMS)):
        got = bench.measured_traffic(profile, "quantize_kernel<true, true, true, true")
        assert got is not None, profile
        rows = [l for l in (root / "profiles" / profile).read_text().splitlines() if l.startswith("quantize_kernel<true, true, true, true")]
        assert rows and any(abs(float(r.split()[-1]) * 1e6 - got) < 1 for r in rows)
        assert 5 * elems <= got <= 1.01 * 5 * elems, (profile, got, 5 * elems)
        text = (root / "profiles" / profile).read_text()
        assert re.search(r"rocprofv3 --pmc FETCH_SIZE", text) and re.search(r"rocprofv3 --pmc WRITE_SIZE", text)
    assert bench.measured_traffic("no_such_file.txt", "quantize_kernel") is None
