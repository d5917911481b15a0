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
    """Uncompressed path, as the reference spells it (collectives.py:12-28): divide by the group size
    for AVG, then ``dist.all_reduce(tensor, op)`` with the caller's op.  (With AVG the reference thus
    divides and then asks the backend for AVG as well; Gloo rejects AVG, so in practice only SUM reaches
    it.  Kept as is: this path is the reference's, not a kernel of this build.)
    A ``SimulatedRing`` group is reduced in place: pre-division for AVG, then the sum."""
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
    dist.all_reduce(tensor, op, group=group)


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
