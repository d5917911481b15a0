"""Wire format and host staging of the ring's messages (src/zeroband/C/csrc/collectives.cpp:140-150):
uint8 codes with tag ``step`` and a 256-entry float32 lookup with tag ``step + 1000``, through pinned
host double buffers, with a host-to-host loopback in place of the neighbour's send / recv."""
import numpy as np
import pytest
import torch

from tests.gpu_util import announce

pytestmark = pytest.mark.gpu


def _inputs(W, n, seed):
    rng = np.random.default_rng(seed)
    return [(rng.standard_normal(n) * 10).astype(np.float32) for _ in range(W)]


def test_message_tags_and_slot_contents(dev):
    from prime_amd import ops, wire

    assert wire.message_tags(7) == (1007, 7) and wire.BUFFER_COUNT == 2
    n = 50_000
    stage = wire.HostStage(dev, n)
    x = torch.randn(n, device=dev)
    announce("host stage round trip")
    codes, lut = ops.uniform_8bit_quantize(x)
    stage.post_send(3, codes, lut)
    h_lut, h_codes = stage.take_send(3)
    assert h_lut.is_pinned() and h_codes.is_pinned() and not h_lut.is_cuda
    assert h_lut.dtype == torch.float32 and h_lut.shape == (256,) and h_codes.dtype == torch.uint8 and h_codes.shape == (n,)
    assert torch.equal(h_codes, codes.cpu()) and torch.equal(h_lut, lut.cpu())
    # the receiving side: host slot -> device slot, usable by a ring step on the current stream
    r_lut, r_codes = stage.recv_buffers(3)
    r_lut.copy_(h_lut)
    r_codes.copy_(h_codes)
    d_codes, d_lut = stage.to_device(3)
    acc = torch.zeros(n, device=dev)
    ops.dequantize_(acc, d_codes, d_lut, True)
    stage.release(3)
    torch.cuda.synchronize()
    assert torch.equal(acc, lut[codes.long()])
    with pytest.raises(RuntimeError, match="posted"):
        wire.HostStage(dev, n).take_send(1)
    with pytest.raises(RuntimeError, match="uint8 codes"):
        stage.post_send(4, torch.cat([codes, codes[:1]]), lut)          # longer than the slot
    # a shorter message (the last chunk of a tensor that 2 W does not divide) travels in a prefix of the slot
    stage.post_send(4, codes[:10], lut)
    lut_h, codes_h = stage.take_send(4)
    assert codes_h.numel() == 10 and torch.equal(codes_h, codes[:10].cpu())
    rl, rc = stage.recv_buffers(4, 10)
    assert rc.numel() == 10


@pytest.mark.parametrize("W,avg", [(1, False), (2, False), (3, True), (4, True), (8, False)])
def test_staged_ring_equals_the_simulated_ring(dev, W, avg):
    # same kernels, same schedule; every message goes GPU -> pinned host -> loopback -> pinned host -> GPU
    from prime_amd import ring, wire

    n = 2 * W * 25_000
    xs = _inputs(W, n, 300 + W)
    direct = [torch.from_numpy(x.copy()).to(dev) for x in xs]
    staged = [torch.from_numpy(x.copy()).to(dev) for x in xs]
    announce(f"staged ring W={W} avg={avg}")
    ring.ring_allreduce_simulated(direct, avg=avg)
    transport = wire.ring_allreduce_staged(staged, avg=avg)
    torch.cuda.synchronize()
    for a, b in zip(direct, staged):
        assert torch.equal(a, b)
    # per rank and phase (W - 1) * BUFFER_COUNT steps send two tensors each
    steps = 2 * W * (W - 1) * 2
    assert transport.messages == 2 * steps
    assert transport.bytes_moved == steps * (n // (2 * W) + 1024)


def test_staged_ring_reuses_its_stages_across_calls(dev):
    from prime_amd import ring, wire

    W, n = 2, 4 * 60_000
    stages = [wire.HostStage(dev, n // (2 * W)) for _ in range(W)]
    for seed in (1, 2, 3):
        xs = _inputs(W, n, seed)
        direct = [torch.from_numpy(x.copy()).to(dev) for x in xs]
        staged = [torch.from_numpy(x.copy()).to(dev) for x in xs]
        ring.ring_allreduce_simulated(direct)
        wire.ring_allreduce_staged(staged, stages=stages)
        torch.cuda.synchronize()
        assert all(torch.equal(a, b) for a, b in zip(direct, staged))
    with pytest.raises(ValueError, match="HostStage"):
        wire.ring_allreduce_staged(staged, stages=stages[:1])


def _free_port() -> int:
    import socket

    with socket.socket() as sock:
        sock.bind(("127.0.0.1", 0))
        return sock.getsockname()[1]


@pytest.mark.parametrize("W,op,pg,n", [(2, "sum", "default", 1_000_000), (4, "sum", "default", 1_000_000), (2, "avg", "newgroup", 1_000_000),
                                       (4, "avg", "default", 1_000_000), (4, "sum", "default", 1_000_001), (2, "avg", "default", 999_999)])
def test_ring_over_a_real_gloo_group_one_process_per_rank(dev, oracle, tmp_path, W, op, pg, n):
    # the reference's own acceptance test (tests/test_c/test_collectives.py:14-68): W processes on
    # localhost, a Gloo group, each rank randn(N) * 10; here every rank's kernels run on the one GPU and
    # only codes + lookup travel (pinned host memory, dist.isend / irecv with the reference's tags).
    # Each rank's result must equal the simulated ring's bit for bit (same kernels, same schedule), which
    # tracks the oracle ring; and the reference's inequality against the exact all-reduce holds.
    import math
    import os
    import subprocess
    import sys
    from pathlib import Path

    from prime_amd import ring

    # N of the reference test (divisible by 2 W, collectives.py:83), and sizes 2 W does not divide: the last chunk is
    # shorter (collectives.cpp:90) and so are the messages that carry it
    seed = 4000 + W
    root = Path(__file__).resolve().parents[1]
    port = _free_port()
    env = dict(os.environ, PYTHONPATH=str(root))
    announce(f"gloo ring W={W} op={op} group={pg} port={port}")
    procs = [subprocess.Popen([sys.executable, "-u", "-m", "tests.ring_worker", str(r), str(W), str(port), str(n), str(seed), op,
                               str(tmp_path)] + (["newgroup"] if pg == "newgroup" else []),
                              cwd=str(root), env=env, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True) for r in range(W)]
    outs = []
    try:
        for pr in procs:
            out, _ = pr.communicate(timeout=150)
            outs.append(out)
    finally:
        for pr in procs:
            if pr.poll() is None:
                pr.kill()
    for r, pr in enumerate(procs):
        assert pr.returncode == 0, f"rank {r} failed:\n{outs[r][-3000:]}"
    xs = [(np.random.default_rng(seed + r).standard_normal(n) * 10).astype(np.float32) for r in range(W)]
    sim = [torch.from_numpy(x.copy()).to(dev) for x in xs]
    ring.ring_allreduce_simulated(sim, avg=(op == "avg"))
    cpu = [x.copy() for x in xs]
    oracle.ring_allreduce_sim(cpu, avg=(op == "avg"))
    torch.cuda.synchronize()
    exact = np.sum(np.stack(xs).astype(np.float64), axis=0) / (W if op == "avg" else 1)
    for r in range(W):
        got = np.load(tmp_path / f"rank{r}.npy")
        assert np.array_equal(got, sim[r].cpu().numpy()), f"rank {r} differs from the simulated ring"
        err_new = np.linalg.norm(got - exact)
        err_old = np.linalg.norm(cpu[r] - exact)
        assert abs(err_new - err_old) / math.sqrt(n) < 0.5            # tests/test_c/test_collectives.py:57
        assert abs(err_new - err_old) / math.sqrt(n) < 0.02


@pytest.mark.parametrize("W", [2, 4])
def test_all_reduce_timing_script_with_uint8_compression(dev, W):
    # scripts/all_reduce.py of the reference with compression "uint8": rand(1, N) per rank, the ranks share
    # the GPU; the sum of W uniform(0, 1) tensors after 8-bit hops stays within a few quantization steps
    from tests.test_host import _run_ranks

    announce(f"all_reduce_bench uint8 W={W}")
    line = _run_ranks(["--size_model", "1000003", "--n_iters", "2", "--compression", "uint8", "--check"], world=W)
    assert line["ranks"] == W and line["compression"] == "uint8"
    assert line["size_model"] == 1000003 - 1000003 % (2 * W)          # src/zeroband/collectives.py:83
    # one hop's step is 6 * rms / 256 of what it carries; W - 1 accumulations and two more round trips
    assert line["rms_error"] < (W + 1) * 6.0 * line["rms_of_sum"] / 256
    assert line["MBps"] > 0
