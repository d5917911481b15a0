"""The all-reduce call site of the reference (src/zeroband/collectives.py:12-42), unchanged in
shape: ``all_reduce(compression, tensor, op, group)`` dispatching on ``Compression``."""
from __future__ import annotations

from typing import Optional

import torch
import torch.distributed as dist

from .config import Compression


def gloo_all_reduce(
    tensor: torch.Tensor,
    op: dist.ReduceOp = dist.ReduceOp.SUM,
    group: Optional[dist.ProcessGroup] = None,
) -> None:
    """Uncompressed path (src/zeroband/collectives.py:12-28): for AVG divide by the group size, then sum.
    The reference divides and then hands its ``op`` on to ``dist.all_reduce``, so with AVG the backend
    is asked to average once more: Gloo rejects that, and a backend that accepts it would divide twice.
    What the reference means - divide, then SUM - is what both branches here do.
    A ``SimulatedRing`` group is reduced in place the same way."""
    from .C.collectives import SimulatedRing

    if isinstance(group, SimulatedRing):
        if op not in [dist.ReduceOp.SUM, dist.ReduceOp.AVG]:
            raise ValueError(f"Unsupported reduce operation {op}. Only SUM and AVG are supported.")
        if op == dist.ReduceOp.AVG:
            for t in group.tensors:
                t.div_(group.size())
        total = group.tensors[0].clone()
        for t in group.tensors[1:]:
            total.add_(t)
        for t in group.tensors:
            t.copy_(total)
        return
    if group is None:
        group = dist.distributed_c10d._get_default_group()
    if op not in [dist.ReduceOp.SUM, dist.ReduceOp.AVG]:
        raise ValueError(f"Unsupported reduce operation {op}. Only SUM and AVG are supported.")
    if op == dist.ReduceOp.AVG:
        tensor.div_(group.size())
    dist.all_reduce(tensor, dist.ReduceOp.SUM, group=group)


def all_reduce(
    compression: Compression,
    tensor: torch.Tensor,
    op: dist.ReduceOp = dist.ReduceOp.SUM,
    group: Optional[object] = None,
) -> None:
    if compression == Compression.UINT8:
        from .C.collectives import ring_allreduce as ring_allreduce_c

        return ring_allreduce_c(tensor, op, group)
    return gloo_all_reduce(tensor, op, group)
