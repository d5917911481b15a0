"""The DiLoCo outer step around the compression path, with everything resident on the GPU.

Counterpart of the parts of ``zeroband.diloco.Diloco`` (src/zeroband/diloco.py) that sit either
side of the compressed all-reduce:

  get_offloaded_param   :147-201  one flat fp32 buffer for the outer parameters, one for the
                                  pseudo-gradient, one view per parameter, one view per layer
                                  bucket (parameters whose names share their first number)
  sync_pseudo_gradient  :78-134   grad = outer - inner, flat buffer / world size, all_reduce per bucket
  outer optimizer       :72-74    torch.optim.SGD(lr=outer_lr, momentum=0.9, nesterov=True)
  sync_inner_model      :137-144  copy the new outer parameters into the model

The reference keeps the outer copy, the gradient and the optimizer state in host memory and
pays a device-to-host copy of every parameter per outer step; with 288 GB of HBM they stay on
the device: the pseudo-gradient is one fused launch per 64 parameters, and the optimizer step
and the copy back to the model are one more.  The retry loop around the all-reduce (:92-126) is
kept, with what it falls back to when every attempt fails (the worker's own pseudo-gradient,
not divided: :127-132); elastic membership and the barrier (:84, :103) belong to the reference's
control plane and are not here: a caller that can rebuild its process group hands
``sync_pseudo_gradient`` a ``regroup`` callable for the retries (:121).

With ``flat_inner=True`` the model's own parameters are moved into a fourth flat buffer laid
out like the other three (each ``param.data`` becomes a view of it).  The pseudo-gradient and
the outer step are then one launch each over the whole model, and the ring can form the
pseudo-gradient of a chunk in the pass that first visits it instead of reading it back
(``prime_amd.ring.ring_allreduce_simulated(..., sources=...)``).
"""
from __future__ import annotations

import re
from functools import lru_cache
from typing import List, Optional, Sequence

import torch
import torch.distributed as dist
from torch import nn

from . import ops
from .collectives import all_reduce
from .config import Compression

OUTER_MOMENTUM = 0.9     # diloco.py:73


@lru_cache(maxsize=None)
def _find_first_number(s: str) -> int:
    """The layer index a parameter name carries, -1 without one (diloco.py:14-21)."""
    match = re.search(r"\d+", s)
    return int(match.group()) if match else -1


class Diloco:
    def __init__(self, outer_lr: float, model: nn.Module, compression: Compression = Compression.UINT8,
                 flat_inner: bool = False):
        self.outer_lr = float(outer_lr)
        self.compression = compression
        self._first_step = True
        self.last_all_reduce_error: Optional[BaseException] = None
        self.inner_flat: Optional[torch.Tensor] = None
        self._init_outer_state(model)
        if flat_inner:
            self._flatten_inner(model)

    @torch.no_grad()
    def _flatten_inner(self, model: nn.Module) -> None:
        """Move the model's parameters into one flat buffer with the layout of the outer copy."""
        self.inner_flat = self.outer_data_flat.clone()
        offset = 0
        for p in self._params(model):
            n = p.numel()
            p.data = self.inner_flat[offset:offset + n].view(p.shape)
            offset += n

    @torch.no_grad()
    def _init_outer_state(self, model: nn.Module) -> None:
        items = [(name, p) for name, p in model.named_parameters() if p.requires_grad]
        if not items:
            raise ValueError("model has no trainable parameter")
        dev = items[0][1].device
        for name, p in items:
            if p.dtype != torch.float32 or p.device != dev or not p.data.is_contiguous():
                raise RuntimeError(f"parameter {name}: contiguous fp32 parameters on one device are required")
        numel = sum(p.numel() for _, p in items)
        self.outer_data_flat = torch.empty(numel, device=dev, dtype=torch.float32)
        self.grad_flat = torch.zeros(numel, device=dev, dtype=torch.float32)
        self.momentum_flat = torch.zeros(numel, device=dev, dtype=torch.float32)
        self._views = []                     # (outer, grad, momentum) flat views per parameter
        cutoffs = []
        offset, prev = 0, None
        for name, p in items:
            if _find_first_number(name) != prev:            # diloco.py:165-167
                cutoffs.append(offset)
                prev = _find_first_number(name)
            n = p.numel()
            sl = slice(offset, offset + n)
            self.outer_data_flat[sl].copy_(p.data.reshape(-1))
            self._views.append((self.outer_data_flat[sl], self.grad_flat[sl], self.momentum_flat[sl]))
            offset += n
        cutoffs.append(offset)
        self.bucket_bounds = list(zip(cutoffs, cutoffs[1:]))
        self.grad_buckets = [self.grad_flat[i:j] for i, j in zip(cutoffs, cutoffs[1:])]      # diloco.py:192-195

    def _params(self, model: nn.Module) -> List[nn.Parameter]:
        ps = [p for p in model.parameters() if p.requires_grad]
        if len(ps) != len(self._views):
            raise RuntimeError("model does not match the one this state was built from")
        return ps

    def _inner_is_flat(self, model: nn.Module) -> bool:
        """True while every parameter still is the view of ``inner_flat`` it was given."""
        if self.inner_flat is None:
            return False
        offset = 0
        for p in self._params(model):
            if p.data.data_ptr() != self.inner_flat.data_ptr() + 4 * offset or not p.data.is_contiguous():
                return False
            offset += p.numel()
        return True

    @torch.no_grad()
    def compute_pseudo_gradient(self, model: nn.Module, world_size: int, fake: bool = False) -> None:
        """grad = (outer - inner) / world_size for every parameter (diloco.py:93-101)."""
        if fake:
            self.grad_flat.zero_()                                   # :95-96
            return
        if self._inner_is_flat(model):
            ops.pseudo_gradient_(self.grad_flat, self.outer_data_flat, self.inner_flat, float(world_size))
            return
        # one launch per 64 parameters instead of one per parameter
        ps = self._params(model)
        ops.pseudo_gradient_segmented_([v[1] for v in self._views], [v[0] for v in self._views], [p.data.view(-1) for p in ps],
                                       float(world_size))

    @torch.no_grad()
    def all_reduce_buckets(self, group: Optional[object]) -> None:
        """One all-reduce per layer bucket (diloco.py:108-110)."""
        for bucket in self.grad_buckets:
            all_reduce(self.compression, bucket, dist.ReduceOp.SUM, group)

    @torch.no_grad()
    def sync_pseudo_gradient(self, model: nn.Module, group: Optional[object], world_size: int, fake: bool = False,
                             retry_all_reduce: int = 1, regroup=None) -> bool:
        """Pseudo-gradient, then the all-reduce of every bucket, tried up to ``retry_all_reduce`` times
        (diloco.py:92-126: the gradient is formed afresh for every attempt, because a failed all-reduce
        leaves the buckets half reduced).  After an attempt that raised, ``regroup()`` (if given) returns the
        group for the next one (:121).  When every attempt has failed the worker keeps its own pseudo-gradient,
        outer - inner, not divided by the world size (:127-132).  Returns whether an all-reduce went through."""
        if retry_all_reduce < 1:
            raise ValueError("retry_all_reduce must be at least 1")
        last = None
        for attempt in range(retry_all_reduce):
            self.compute_pseudo_gradient(model, world_size, fake=fake)
            try:
                self.all_reduce_buckets(group)
                return True
            except Exception as e:      # the reference catches everything here (:119)
                last = e
                if regroup is not None and attempt + 1 < retry_all_reduce:
                    group = regroup()
        self.compute_pseudo_gradient(model, 1, fake=fake)
        self.last_all_reduce_error = last
        return False

    @torch.no_grad()
    def outer_step(self, model: nn.Module) -> None:
        """outer_optimizer.step() and sync_inner_model (diloco.py:212-215), one launch per 64 parameters
        (one for the whole model when the inner parameters are flat)."""
        if self._inner_is_flat(model):
            ops.outer_sgd_nesterov_(self.outer_data_flat, self.momentum_flat, self.grad_flat, self.inner_flat, self.outer_lr,
                                    OUTER_MOMENTUM, self._first_step)
            self._first_step = False
            return
        ps = self._params(model)
        ops.outer_sgd_nesterov_segmented_([v[0] for v in self._views], [v[2] for v in self._views], [v[1] for v in self._views],
                                          [p.data.view(-1) for p in ps], self.outer_lr, OUTER_MOMENTUM, self._first_step)
        self._first_step = False

    @torch.no_grad()
    def step(self, model: nn.Module, group: Optional[object] = None, world_size: Optional[int] = None, fake: bool = False,
             retry_all_reduce: int = 1, regroup=None) -> None:
        """The whole outer step of one worker (diloco.py:203-215).  With ``retry_all_reduce`` > 1 a failing
        all-reduce is tried again as the reference tries it; with the default an exception propagates."""
        if world_size is None:
            world_size = group.size() if group is not None else dist.get_world_size()
        if retry_all_reduce > 1 or regroup is not None:
            self.sync_pseudo_gradient(model, group, world_size, fake=fake, retry_all_reduce=retry_all_reduce, regroup=regroup)
        else:
            self.compute_pseudo_gradient(model, world_size, fake=fake)
            self.all_reduce_buckets(group)
        self.outer_step(model)


@torch.no_grad()
def step_simulated_workers(workers: Sequence[Diloco], models: Sequence[nn.Module], fake: bool = False,
                           coded_gather: bool = True) -> None:
    """The outer step of W workers that live in one process on one GPU: every worker forms its
    pseudo-gradient, each layer bucket goes through the ring all-reduce of W simulated ranks, and
    every worker applies the outer optimizer."""
    from .C.collectives import SimulatedRing

    W = len(workers)
    lazy = (not fake and workers[0].compression == Compression.UINT8
            and all(w._inner_is_flat(m) for w, m in zip(workers, models))
            and all((j - i) % (2 * W) == 0 for i, j in workers[0].bucket_bounds))
    if lazy:
        # the pseudo-gradient of a chunk is formed in the ring pass that first visits it; with
        # coded_gather the all-gather stays in the code domain and the outer step dequantizes
        from . import ring

        for b, (i, j) in enumerate(workers[0].bucket_bounds):
            final = ring.ring_allreduce_simulated([w.grad_buckets[b] for w in workers], avg=False,
                                                  sources=[(w.outer_data_flat[i:j], w.inner_flat[i:j]) for w in workers],
                                                  world_size=float(W), keep_codes=coded_gather)
            if coded_gather:
                csz = (j - i) // (2 * W)
                for w, chunks in zip(workers, final):
                    for c, (codes, lut) in enumerate(chunks):
                        sl = slice(i + c * csz, i + (c + 1) * csz)
                        ops.outer_sgd_nesterov_codes_(w.outer_data_flat[sl], w.momentum_flat[sl], codes, lut, w.inner_flat[sl],
                                                      w.outer_lr, OUTER_MOMENTUM, w._first_step)
        for w, m in zip(workers, models):
            if coded_gather:
                w._first_step = False
            else:
                w.outer_step(m)
        return
    for w, m in zip(workers, models):
        w.compute_pseudo_gradient(m, W, fake=fake)
    for b in range(len(workers[0].grad_buckets)):
        bucket = [w.grad_buckets[b] for w in workers]
        all_reduce(workers[0].compression, bucket[0], dist.ReduceOp.SUM, SimulatedRing(bucket))
    for w, m in zip(workers, models):
        w.outer_step(m)
