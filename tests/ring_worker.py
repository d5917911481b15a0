"""One rank of a ring all-reduce over a real Gloo group, run as a child process by
tests/test_gpu_wire.py (the way tests/test_c/test_collectives.py:14-68 of the reference forks one
process per rank on localhost):

    python -m tests.ring_worker RANK WORLD PORT N SEED OP OUT_DIR

Every rank puts its tensor on cuda:0, calls all_reduce(Compression.UINT8, t, op, group) and saves
the result as OUT_DIR/rank<RANK>.npy.
"""
import datetime
import os
import sys

import numpy as np


def main() -> int:
    rank, world, port, n, seed = (int(a) for a in sys.argv[1:6])
    op_name, out_dir = sys.argv[6], sys.argv[7]
    os.environ.update(RANK=str(rank), WORLD_SIZE=str(world), MASTER_ADDR="127.0.0.1", MASTER_PORT=str(port),
                      GLOO_SOCKET_IFNAME="lo")
    import torch
    import torch.distributed as dist

    from prime_amd.collectives import Compression, all_reduce

    print(f"[gpu-case] ring worker rank {rank}/{world} n={n} op={op_name}", flush=True)
    dist.init_process_group("gloo", rank=rank, world_size=world, timeout=datetime.timedelta(seconds=60))
    try:
        rng = np.random.default_rng(seed + rank)
        x = (rng.standard_normal(n) * 10).astype(np.float32)             # tests/test_c/test_collectives.py:39
        t = torch.from_numpy(x).to("cuda:0")
        op = dist.ReduceOp.AVG if op_name == "avg" else dist.ReduceOp.SUM
        group = dist.new_group(list(range(world)), backend="gloo") if len(sys.argv) > 8 and sys.argv[8] == "newgroup" else None
        all_reduce(Compression.UINT8, t, op, group)
        torch.cuda.synchronize()
        np.save(os.path.join(out_dir, f"rank{rank}.npy"), t.cpu().numpy())
    finally:
        dist.destroy_process_group()
    return 0


if __name__ == "__main__":
    sys.exit(main())
