"""What crosses the wire in the ring, and the pinned host buffers between the GPU and a host
transport.

The reference sends, per step, two tensors to the next rank (src/zeroband/C/csrc/collectives.cpp:140-150):

    lookup   float32[256]            tag step + 1000
    codes    uint8[chunk numel]      tag step

through ``group->send`` / ``group->recv`` of a c10d process group (Gloo: host memory), with
BUFFER_COUNT = 2 slots in flight (:6, :118-122).  Its tensors already live in host memory.  Here
codes and lookup are produced on the GPU, so each rank keeps

    send slots   pinned host memory, filled by asynchronous device-to-host copies on a copy stream
    recv slots   pinned host memory the transport writes into, drained by host-to-device copies
    device recv  the buffers the ring-step kernels read

and only uint8 codes + 1 KiB cross PCIe (a quarter of the fp32 chunk).  Copies run on their own
HIP stream of default priority and are ordered against the compute stream with events, so the
copy of step s overlaps the kernels of step s + 1, as the reference overlaps its sends with
the next quantization.

Two transports sit behind the stage.  ``ring_allreduce_group`` is the reference's own: one process
per rank, ``dist.isend`` / ``dist.irecv`` of the pinned host slots over a c10d group with a host
(Gloo) backend, the reference's tags and its two slots in flight; the ranks may share one GPU.
``Loopback`` stands in for the neighbour's ``send`` / ``recv`` pair inside one process (W simulated
ranks) by copying host slot to host slot, which runs the same schedule through the staging path
and times the PCIe side without a second process.
"""
from __future__ import annotations

from typing import Dict, List, Optional, Sequence, Tuple

import torch
import torch.distributed as dist

from . import ops
from .ring import BUFFER_COUNT, _check_ring_inputs, chunk_bounds

LOOKUP_TAG_OFFSET = 1000      # collectives.cpp:141,144
N_BINS = ops.N_BINS


def message_tags(step: int) -> Tuple[int, int]:
    """(tag of the lookup table, tag of the codes) for one step (collectives.cpp:141,147)."""
    return step + LOOKUP_TAG_OFFSET, step


class HostStage:
    """One rank's staging buffers for chunks of ``chunk_numel`` elements."""

    def __init__(self, device: torch.device, chunk_numel: int, depth: int = BUFFER_COUNT):
        self.device = torch.device(device)
        self.chunk_numel = int(chunk_numel)
        self.depth = int(depth)
        self.copy_stream = torch.cuda.Stream(self.device)

        def pinned(shape, dtype):
            return torch.empty(shape, dtype=dtype, pin_memory=True)

        with torch.cuda.device(self.device):
            self.send_codes = [pinned(self.chunk_numel, torch.uint8) for _ in range(self.depth)]
            self.send_lut = [pinned(N_BINS, torch.float32) for _ in range(self.depth)]
            self.recv_codes = [pinned(self.chunk_numel, torch.uint8) for _ in range(self.depth)]
            self.recv_lut = [pinned(N_BINS, torch.float32) for _ in range(self.depth)]
            self.dev_codes = [torch.empty(self.chunk_numel, dtype=torch.uint8, device=self.device) for _ in range(self.depth)]
            self.dev_lut = [torch.empty(N_BINS, dtype=torch.float32, device=self.device) for _ in range(self.depth)]
        self._d2h_done: List[Optional[torch.cuda.Event]] = [None] * self.depth
        self._h2d_done: List[Optional[torch.cuda.Event]] = [None] * self.depth
        self._consumed: List[Optional[torch.cuda.Event]] = [None] * self.depth
        self._keep: List[tuple] = [()] * self.depth       # device tensors a copy in flight still reads
        self._sent_numel: List[int] = [self.chunk_numel] * self.depth

    # ---- sending -------------------------------------------------------------------------------
    def post_send(self, step: int, codes: torch.Tensor, lut: torch.Tensor) -> None:
        """Start the device-to-host copy of one message; the kernels that produced it are on the
        current stream.  The slot must have been taken by the transport (``take_send``) before it is
        reused, BUFFER_COUNT steps later."""
        if codes.numel() > self.chunk_numel or codes.dtype != torch.uint8 or lut.numel() != N_BINS or lut.dtype != torch.float32:
            raise RuntimeError("post_send: a message is uint8 codes of at most the chunk size and 256 float32 lookup entries")
        slot = step % self.depth
        ready = torch.cuda.current_stream(self.device).record_event()
        self.copy_stream.wait_event(ready)
        with torch.cuda.stream(self.copy_stream):
            self.send_lut[slot].copy_(lut.view(-1), non_blocking=True)
            self.send_codes[slot][:codes.numel()].copy_(codes.view(-1), non_blocking=True)
            self._d2h_done[slot] = self.copy_stream.record_event()
        self._keep[slot] = (codes, lut)
        self._sent_numel[slot] = codes.numel()

    def take_send(self, step: int) -> Tuple[torch.Tensor, torch.Tensor]:
        """Block until the message of ``step`` is in host memory; returns (lookup, codes), the two
        host tensors to hand to ``send`` with ``message_tags(step)``."""
        slot = step % self.depth
        ev = self._d2h_done[slot]
        if ev is None:
            raise RuntimeError(f"no message was posted for step {step}")
        ev.synchronize()
        self._keep[slot] = ()
        return self.send_lut[slot], self.send_codes[slot][:self._sent_numel[slot]]

    # ---- receiving -----------------------------------------------------------------------------
    def recv_buffers(self, step: int, numel: Optional[int] = None) -> Tuple[torch.Tensor, torch.Tensor]:
        """(lookup, codes) host tensors for ``recv`` with ``message_tags(step)``; ``numel`` codes (the
        chunk size unless the message is the shorter last chunk of a tensor).  Blocks until the
        host-to-device copy that last read this slot has finished."""
        slot = step % self.depth
        if self._h2d_done[slot] is not None:
            self._h2d_done[slot].synchronize()
        k = self.chunk_numel if numel is None else int(numel)
        return self.recv_lut[slot], self.recv_codes[slot][:k]

    def to_device(self, step: int, numel: Optional[int] = None) -> Tuple[torch.Tensor, torch.Tensor]:
        """Start the host-to-device copy of the received message of ``step`` (``numel`` codes) and order
        the current stream after it; returns (codes, lookup) on the device."""
        slot = step % self.depth
        k = self.chunk_numel if numel is None else int(numel)
        if self._consumed[slot] is not None:
            self.copy_stream.wait_event(self._consumed[slot])      # the kernels that read this device slot last
        with torch.cuda.stream(self.copy_stream):
            self.dev_lut[slot].copy_(self.recv_lut[slot], non_blocking=True)
            self.dev_codes[slot][:k].copy_(self.recv_codes[slot][:k], non_blocking=True)
            self._h2d_done[slot] = self.copy_stream.record_event()
        torch.cuda.current_stream(self.device).wait_event(self._h2d_done[slot])
        return self.dev_codes[slot][:k], self.dev_lut[slot]

    def release(self, step: int) -> None:
        """The kernels reading the device slot of ``step`` have been enqueued on the current stream."""
        self._consumed[step % self.depth] = torch.cuda.current_stream(self.device).record_event()


class Loopback:
    """Stand-in for the neighbour-to-neighbour ``send`` / ``recv`` pair: host memory to host
    memory inside one process.  ``bytes_moved`` counts what a real transport would carry."""

    def __init__(self):
        self.bytes_moved = 0
        self.messages = 0

    def deliver(self, src: HostStage, dst: HostStage, step: int) -> None:
        lut, codes = src.take_send(step)
        rl, rc = dst.recv_buffers(step, codes.numel())
        rl.copy_(lut)
        rc.copy_(codes)
        self.bytes_moved += lut.numel() * 4 + codes.numel()
        self.messages += 2            # two tensors per step, tags step + 1000 and step


def ring_allreduce_staged(tensors: Sequence[torch.Tensor], avg: bool = False, transport: Optional[Loopback] = None,
                          stages: Optional[Sequence[HostStage]] = None) -> Loopback:
    """``ring_allreduce`` (collectives.cpp:76-230) for ``len(tensors)`` simulated ranks with every
    message taking the path of a host transport: GPU -> pinned host (sender) -> transport ->
    pinned host (receiver) -> GPU.  Same kernels and schedule as
    ``prime_amd.ring.ring_allreduce_simulated``, so the results are identical to it."""
    W = len(tensors)
    n = _check_ring_inputs(tensors)
    nb = BUFFER_COUNT * W
    bounds = chunk_bounds(n, W)
    csz = bounds[0][1] - bounds[0][0]              # the largest chunk: what the buffers are sized for (collectives.cpp:104)
    flats = [t.view(-1) for t in tensors]
    dev = flats[0].device
    transport = transport or Loopback()
    if stages is None:
        stages = [HostStage(dev, csz) for _ in range(W)]
    if len(stages) != W or any(s.chunk_numel != csz for s in stages):
        raise ValueError("one HostStage per rank, sized for the chunk, is needed")

    def chunk(r: int, c: int) -> torch.Tensor:
        return flats[r][bounds[c][0]:bounds[c][1]]

    own: Dict[Tuple[int, int], Tuple[torch.Tensor, torch.Tensor]] = {}
    for phase in (1, 2):
        arrived = [set() for _ in range(W)]
        for step in range(1, nb + 1):
            posted = []
            for r in range(W):
                c = ((r * BUFFER_COUNT - step) if phase == 1 else (r * BUFFER_COUNT + BUFFER_COUNT - step)) % nb   # :116 / :192
                ch = chunk(r, c)
                got = (step - BUFFER_COUNT) in arrived[r]
                sending = step <= (W - 1) * BUFFER_COUNT                                                        # :136 / :212
                out = None
                if got:
                    arrived[r].discard(step - BUFFER_COUNT)
                    codes_in, lut_in = stages[r].to_device(step - BUFFER_COUNT, ch.numel())
                    if sending:
                        out = (ops.ring_reduce_step if phase == 1 else ops.ring_gather_step)(ch, codes_in, lut_in)
                    elif phase == 1:
                        own[(r, c)] = ops.ring_reduce_div_step(ch, codes_in, lut_in, float(W) if avg else 1.0)
                    else:
                        ops.dequantize_(ch, codes_in, lut_in, False)
                    stages[r].release(step - BUFFER_COUNT)
                elif sending and (r, c) in own:
                    out = ops.ring_gather_step(ch, *own.pop((r, c)))
                elif sending:
                    out = ops.uniform_8bit_quantize(ch, False)
                if out is not None:
                    stages[r].post_send(step, out[0], out[1])
                    posted.append(r)
            for r in posted:                       # the transport: rank r -> rank r + 1
                transport.deliver(stages[r], stages[(r + 1) % W], step)
                arrived[(r + 1) % W].add(step)
        if phase == 1 and W == 1:
            for i in range(BUFFER_COUNT):
                ch = chunk(0, i)
                codes, lut = ops.uniform_8bit_quantize(ch, True)
                ops.dequantize_(ch, codes, lut, False)
    assert not own
    return transport


_stages: Dict[Tuple[int, int, int], HostStage] = {}
_STAGE_CACHE_MAX = 8


def _stage_for(device: torch.device, chunk_numel: int, group) -> HostStage:
    """One HostStage per (device, chunk size, group), kept: pinned allocations are slow and the per-layer
    buckets of a model repeat a handful of sizes.  The cache holds at most _STAGE_CACHE_MAX stages (the
    least recently used one is dropped: each holds four pinned and two device chunk buffers), and a
    stage is never shared by two groups.  Calls on one group are expected one at a time, as a ring
    all-reduce is; two threads driving the same group concurrently would share its slots."""
    idx = device.index if device.index is not None else torch.cuda.current_device()
    key = (idx, int(chunk_numel), id(group))
    st = _stages.pop(key, None)
    if st is None:
        st = HostStage(torch.device("cuda", idx), chunk_numel)
        while len(_stages) >= _STAGE_CACHE_MAX:
            _stages.pop(next(iter(_stages)))
    _stages[key] = st                 # most recently used last
    return st


def ring_allreduce_group(tensor: torch.Tensor, avg: bool, group) -> None:
    """``ring_allreduce`` (collectives.cpp:76-230) for THIS rank of a real process group whose backend
    moves host memory (Gloo).  Schedule, tags and buffering are the reference's: at step s the rank
    waits for the four transfers posted at step s - 2 (:118-122), folds the received message into
    chunk c(s) on the GPU, and if s <= 2 (W - 1) quantizes that chunk and posts
    ``isend(lookup, tag s + 1000)``, ``irecv(lookup)``, ``isend(codes, tag s)``, ``irecv(codes)`` with
    the next and previous rank (:140-150, :217-227).  Messages live in the two pinned host slots of a
    ``HostStage``; only codes and lookup cross PCIe.  In place; every rank must call it."""
    W = group.size()
    rank = dist.get_rank(group)
    flat = tensor.view(-1)
    n = _check_ring_inputs([flat] * W)
    nb = BUFFER_COUNT * W
    bounds = chunk_bounds(n, W)
    csz = bounds[0][1] - bounds[0][0]              # the largest chunk (collectives.cpp:104)
    stage = _stage_for(flat.device, csz, group)
    dst = dist.get_global_rank(group, (rank + 1) % W)                    # :111
    src = dist.get_global_rank(group, (rank - 1 + W) % W)               # :112

    def chunk(c: int) -> torch.Tensor:
        return flat[bounds[c][0]:bounds[c][1]]

    def chunk_of(r: int, phase: int, step: int) -> int:
        return ((r * BUFFER_COUNT - step) if phase == 1 else (r * BUFFER_COUNT + BUFFER_COUNT - step)) % nb     # :116 / :192

    own: Dict[int, Tuple[torch.Tensor, torch.Tensor]] = {}
    for phase in (1, 2):
        works: Dict[int, list] = {}
        pending: Optional[int] = None      # step whose message is on its way to the pinned send slot, not yet handed to the transport

        def hand_over() -> None:
            # the host waits for the device-to-host copy only here, after the next step's kernels are enqueued:
            # the copy of step s runs beside the kernels of step s + 1
            nonlocal pending
            if pending is None:
                return
            s_ = pending
            pending = None
            lut_h, codes_h = stage.take_send(s_)                         # the message is in pinned host memory
            # what arrives is the previous rank's chunk of the same step: its size is known here without being sent
            prev_c = chunk_of((rank - 1 + W) % W, phase, s_)
            rl, rc = stage.recv_buffers(s_, bounds[prev_c][1] - bounds[prev_c][0])
            lut_tag, codes_tag = message_tags(s_)
            works[s_] = [dist.isend(lut_h, dst, group=group, tag=lut_tag), dist.irecv(rl, src, group=group, tag=lut_tag),
                         dist.isend(codes_h, dst, group=group, tag=codes_tag), dist.irecv(rc, src, group=group, tag=codes_tag)]

        for step in range(1, nb + 1):
            c = ((rank * BUFFER_COUNT - step) if phase == 1 else (rank * BUFFER_COUNT + BUFFER_COUNT - step)) % nb   # :116 / :192
            ch = chunk(c)
            sending = step <= (W - 1) * BUFFER_COUNT                                                              # :136 / :212
            out = None
            if (step - BUFFER_COUNT) in works:
                for w in works.pop(step - BUFFER_COUNT):                 # :118-122
                    w.wait()
                codes_in, lut_in = stage.to_device(step - BUFFER_COUNT, ch.numel())
                if sending:
                    out = (ops.ring_reduce_step if phase == 1 else ops.ring_gather_step)(ch, codes_in, lut_in)
                elif phase == 1:
                    own[c] = ops.ring_reduce_div_step(ch, codes_in, lut_in, float(W) if avg else 1.0)
                else:
                    ops.dequantize_(ch, codes_in, lut_in, False)
                stage.release(step - BUFFER_COUNT)
            elif sending and c in own:
                out = ops.ring_gather_step(ch, *own.pop(c))
            elif sending:
                out = ops.uniform_8bit_quantize(ch, False)
            hand_over()                                                  # the message of the step before
            if out is not None:
                stage.post_send(step, out[0], out[1])
                pending = step
        hand_over()
        assert not works
    assert not own
