"""Drop-in for ``zeroband.C.collectives`` (src/zeroband/C/collectives.py:23-35):
``ring_allreduce(tensor, op, group)`` with the per-hop compute on the GPU.

Groups it accepts:

* a real c10d process group with a host (Gloo) backend, as the reference uses
  (``ProcessGroupGloo``, C/collectives.py:30-35): one process per rank, messages through pinned host
  memory and ``dist.isend`` / ``dist.irecv`` (``prime_amd.wire.ring_allreduce_group``); the ranks may
  share one GPU.  A group of size 1 is the single rank's quantize / dequantize round trip;
* a ``SimulatedRing`` holding the tensors of W ranks on one device: the full schedule runs
  in one process (``prime_amd.ring.ring_allreduce_simulated``);
* ``FakeProcessGroup``: returns at once, as the reference does (C/collectives.py:32-33).

A group whose backend cannot move host tensors (NCCL / RCCL only) raises NotImplementedError: a
device-to-device transport needs a second GPU and is not part of this build.
"""
from __future__ import annotations

from typing import List, Optional

import torch
import torch.distributed as dist

from .. import _lib, ring

_lib.load()


class SimulatedRing:
    """W ranks of a ring all-reduce living in one process: ``tensors[r]`` is rank r's buffer.
    Passing it as ``group`` reduces all of them in place; ``tensor`` must be one of them."""

    def __init__(self, tensors: List[torch.Tensor]):
        self.tensors = list(tensors)

    def size(self) -> int:
        return len(self.tensors)


def _check_op(op) -> bool:
    """True for AVG; SUM and AVG only, as collectives.cpp:83 checks."""
    if op == dist.ReduceOp.SUM:
        return False
    if op == dist.ReduceOp.AVG:
        return True
    raise RuntimeError("Unsupported reduce operation. Only SUM and AVG are supported.")


def ring_allreduce(
    tensor: torch.Tensor,
    op: dist.ReduceOp = dist.ReduceOp.SUM,
    group: Optional[object] = None,
) -> None:
    avg = _check_op(op)
    if isinstance(group, SimulatedRing):
        if not any(t is tensor for t in group.tensors):
            raise ValueError("tensor is not one of the simulated ring's rank buffers")
        ring.ring_allreduce_simulated(group.tensors, avg=avg)
        return
    if group is None:
        group = dist.distributed_c10d._get_default_group()
    try:
        from torch.testing._internal.distributed.fake_pg import FakeProcessGroup
    except Exception:  # the class is a torch-internal test helper
        FakeProcessGroup = ()
    if FakeProcessGroup and isinstance(group, FakeProcessGroup):
        return
    if group.size() == 1:
        ring.ring_allreduce_single(tensor, avg=avg)
        return
    backend = str(dist.get_backend(group)).lower()
    if "gloo" not in backend:
        raise NotImplementedError(
            f"ring_allreduce moves its messages through host memory and needs a Gloo group (got backend {backend!r}); "
            "a device-to-device transport is not part of this single-GPU build")
    from .. import wire

    wire.ring_allreduce_group(tensor, avg, group)
