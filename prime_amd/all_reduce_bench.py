"""Timing of ``all_reduce(compression, tensor, op)`` between the ranks of a Gloo group, the
measurement the reference ships as scripts/all_reduce.py:33-60 (same knobs: the element count, the
number of timed iterations, the compression; same figures: mean seconds per iteration and
``size_model * 4 / 1e6 / seconds`` MB/s).  One process per rank:

    python -m torch.distributed.run --nnodes=1 --nproc-per-node 2 --master-addr 127.0.0.1 \\
        --master-port 29511 -m prime_amd.all_reduce_bench --size_model 10000000 --n_iters 4 --compression uint8

With ``--compression uint8`` the tensor lives on the GPU (every rank of one host on ``--device``),
the kernels of the ring run there and only codes + lookup cross the Gloo group through pinned host
memory; with ``no`` the tensor stays on the host and goes through ``dist.all_reduce`` as in the
reference.  ``--check`` compares the result with the exact sum (the reference's test bound,
tests/test_c/test_collectives.py:57, needs the other ranks' inputs, which are seeded by rank).
"""
from __future__ import annotations

import argparse
import datetime
import json
import math
import sys
import time


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(description=__doc__.split("\n\n")[0])
    ap.add_argument("--size_model", type=int, default=int(1e7))                 # scripts/all_reduce.py:29
    ap.add_argument("--n_iters", type=int, default=4)                           # :30
    ap.add_argument("--compression", choices=["no", "uint8"], default="no")     # :31
    ap.add_argument("--device", default="cuda:0", help="where a uint8-compressed tensor lives")
    ap.add_argument("--check", action="store_true", help="compare the last result with the exact sum of the ranks' inputs")
    args = ap.parse_args(argv)

    import torch
    import torch.distributed as dist

    from .collectives import Compression, all_reduce

    dist.init_process_group(backend="gloo", timeout=datetime.timedelta(seconds=120))     # scripts/all_reduce.py:66
    try:
        rank, world = dist.get_rank(), dist.get_world_size()
        compression = Compression(args.compression)
        n = args.size_model
        if compression == Compression.UINT8 and n % (2 * world):
            n -= n % (2 * world)                                                # src/zeroband/collectives.py:83
        gen = torch.Generator().manual_seed(1234 + rank)
        host = torch.rand(1, n, generator=gen)                                  # scripts/all_reduce.py:37
        dev = torch.device(args.device if compression == Compression.UINT8 else "cpu")
        mat = host.to(dev)

        def sync():
            if dev.type == "cuda":
                torch.cuda.synchronize(dev)

        all_reduce(compression, mat.clone(), op=dist.ReduceOp.SUM)              # untimed: workspaces, pinned stages, connections
        sync()
        times = []
        for _ in range(args.n_iters):
            work = mat.clone()
            sync()
            dist.barrier()
            t0 = time.perf_counter()
            all_reduce(compression, work, op=dist.ReduceOp.SUM)
            sync()
            times.append(time.perf_counter() - t0)
        seconds = sum(times) / len(times)
        line = {"ranks": world, "size_model": n, "compression": compression.value, "n_iters": args.n_iters,
                "seconds_per_iteration": seconds, "MBps": n * 4 / 1e6 / seconds}       # scripts/all_reduce.py:55
        if args.check:
            exact = torch.zeros(1, n, dtype=torch.float64)
            for r in range(world):
                exact += torch.rand(1, n, generator=torch.Generator().manual_seed(1234 + r)).double()
            err = (work.cpu().double() - exact).norm().item() / math.sqrt(n)
            line["rms_error"] = err
            line["rms_of_sum"] = exact.norm().item() / math.sqrt(n)
        if rank == 0:
            print(json.dumps(line), flush=True)
    finally:
        dist.destroy_process_group()
    return 0


if __name__ == "__main__":
    sys.exit(main())
