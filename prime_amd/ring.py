"""The ring all-reduce's compute, run on one GPU for W simulated ranks.

The reference's ``ring_allreduce`` (src/zeroband/C/csrc/collectives.cpp:76-230; readable twin
src/zeroband/collectives.py:53-192) splits each rank's tensor into 2 W chunks and passes
uint8 codes plus a 256-entry lookup round the ring.  What a rank computes per received
message is fixed by the schedule and independent of the transport:

  reduce-scatter   chunk += lut[codes]; (codes, lut) = uniform_8bit_quantize(chunk)   :124-138
  own chunks       [chunk /= W]; chunk = lut[codes] of its own quantization          :155-173
  all-gather       chunk = lut[codes]; re-quantize before forwarding                 :194-215

Here every "rank" is a tensor on the same device and a send is a hand-over of the
(codes, lut) pair; the kernels are the ones a real ring over RCCL or TCP would run.
"""
from __future__ import annotations

from typing import List, Optional, Sequence, Tuple

import torch

from . import ops

BUFFER_COUNT = 2   # collectives.cpp:6


def ring_hops(chunks: Sequence[torch.Tensor]) -> Tuple[torch.Tensor, torch.Tensor]:
    """One chunk's trip through the reduce-scatter phase: ``chunks[r]`` is what the r-th rank
    on the path holds.  chunks[0] is quantized; each later rank accumulates the received
    codes into its chunk (in place) and requantizes.  Returns the last (codes, lut)."""
    codes, lut = ops.uniform_8bit_quantize(chunks[0], False)
    for acc in chunks[1:]:
        codes, lut = ops.ring_reduce_step(acc, codes, lut)
    return codes, lut


def _check_ring_inputs(tensors: Sequence[torch.Tensor]) -> int:
    if len(tensors) == 0:
        raise ValueError("at least one rank is needed")
    n = tensors[0].numel()
    for t in tensors:
        if t.dtype != torch.float32:
            raise RuntimeError(f"expected scalar type Float but found {t.dtype}")
        if t.numel() != n or t.device != tensors[0].device:
            raise ValueError("all simulated ranks must hold tensors of one size on one device")
        if not t.is_contiguous():
            raise RuntimeError("ring all-reduce works in place and needs contiguous tensors")
    chunk_bounds(n, len(tensors))
    return n


def chunk_bounds(n: int, world_size: int) -> List[Tuple[int, int]]:
    """[lo, hi) of the 2 * world_size chunks ``flat.chunk(2 * world_size)`` cuts a tensor of n elements
    into (collectives.cpp:89-90): pieces of ceil(n / 2W) elements, the last one shorter when 2W does
    not divide n.  The reference's C++ takes any n that yields all 2W chunks (its Python twin asserts
    divisibility, src/zeroband/collectives.py:83); when ``torch.chunk`` returns fewer pieces the C++
    would index past its chunk list, and this raises instead."""
    nb = BUFFER_COUNT * world_size
    size = -(-n // nb) if n else 0
    bounds = [(lo, min(n, lo + size)) for lo in range(0, n, size)] if size else []
    if len(bounds) != nb:
        raise ValueError(f"Tensor size must split into {nb} chunks: torch.chunk cuts {n} elements into {len(bounds)} pieces of "
                         f"{size} (pad the tensor to a multiple of {nb} elements)")
    return bounds


def ring_allreduce_simulated(tensors: Sequence[torch.Tensor], avg: bool = False,
                             sources: Optional[Sequence[Tuple[torch.Tensor, torch.Tensor]]] = None,
                             world_size: Optional[float] = None,
                             keep_codes: bool = False) -> Optional[List[List[Tuple[torch.Tensor, torch.Tensor]]]]:
    """The whole of ``ring_allreduce`` for ``len(tensors)`` ranks, in place, in lock step.

    A message posted at step s is consumed at step s + 2 (BUFFER_COUNT receive slots,
    collectives.cpp:118-122), which lock-stepping the ranks reproduces exactly.

    With ``sources`` = one (outer, inner) pair of flat tensors per rank, ``tensors[r]`` need not
    hold anything yet: rank r's pseudo-gradient (outer - inner) / world_size (diloco.py:93-101) is
    formed chunk by chunk in the reduce-scatter, where every chunk of a rank is visited exactly
    once, and the result is what the all-reduce of the materialized pseudo-gradients gives.

    With ``keep_codes`` the all-gather stays in the code domain: a rank's final value of a chunk
    is ``lut[codes]`` of the message it received (or of its own quantization), so the fp32 chunk is
    not written; what is forwarded, ``uniform_8bit_quantize(lut[codes])`` (:215), is computed from
    the codes alone (``ops.requantize_codes``).  Returns ``result[r][c] = (codes, lut)`` for every
    rank r and chunk c; ``tensors`` then hold stale reduce-scatter values and the caller
    dequantizes where it needs fp32 (``ops.dequantize_``, ``ops.outer_sgd_nesterov_codes_``)."""
    W = len(tensors)
    n = _check_ring_inputs(tensors)
    if sources is not None:
        if len(sources) != W:
            raise ValueError("one (outer, inner) pair per simulated rank is needed")
        for o, i in sources:
            if o.numel() != n or i.numel() != n:
                raise ValueError("outer and inner must have the size of the rank's tensor")
        if world_size is None:
            world_size = float(W)
    nb = BUFFER_COUNT * W
    bounds = chunk_bounds(n, W)
    flats = [t.view(-1) for t in tensors]

    def chunk(r: int, c: int) -> torch.Tensor:
        return flats[r][bounds[c][0]:bounds[c][1]]

    def touch(r: int, c: int, msg, divisor: float):
        # first and only visit of chunk c by rank r in the reduce-scatter, pseudo-gradient included
        o, i = sources[r]
        sl = slice(*bounds[c])
        return ops.ring_first_touch_(chunk(r, c), o.view(-1)[sl], i.view(-1)[sl], float(world_size),
                                     None if msg is None else msg[0], None if msg is None else msg[1], divisor)

    own: dict = {}     # (rank, chunk) -> (codes, lut) of the rank's reduced chunk, not yet written back
    final: List[List] = [[None] * nb for _ in range(W)]
    div = float(W) if avg else 1.0
    for phase in (1, 2):
        inbox: List[dict] = [dict() for _ in range(W)]
        for step in range(1, nb + 1):
            posted = []
            # What every rank does in this step.  The W ranks' work of one kind is independent, so it goes to
            # the device as one segmented call (three launches for all ranks) instead of three launches per rank.
            batch: dict = {}       # kind -> list of (rank, chunk index, chunk, message)
            for r in range(W):
                if phase == 1:
                    c = (r * BUFFER_COUNT - step) % nb                      # collectives.cpp:116
                else:
                    c = (r * BUFFER_COUNT + BUFFER_COUNT - step) % nb       # :192
                ch = chunk(r, c)
                msg = inbox[r].pop(step - BUFFER_COUNT, None)
                sending = step <= (W - 1) * BUFFER_COUNT                    # :136 / :212
                if phase == 1 and sources is not None and (msg is not None or sending):
                    pair = touch(r, c, msg, div if not sending else 1.0)
                    if sending:
                        posted.append(((r + 1) % W, step, pair[0], pair[1]))
                    else:
                        own[(r, c)] = pair
                elif phase == 2 and keep_codes and (msg is not None or (r, c) in own):
                    pair = msg if msg is not None else own.pop((r, c))
                    final[r][c] = pair
                    if sending:
                        codes, lut = ops.requantize_codes(pair[0], pair[1])     # :215 without the fp32 chunk
                        posted.append(((r + 1) % W, step, codes, lut))
                elif msg is not None and sending:
                    # :128-138 fused (phase 1) / :204-215 fused (phase 2)
                    batch.setdefault(ops.SEG_REDUCE if phase == 1 else ops.SEG_GATHER, []).append((r, c, ch, msg))
                elif msg is not None and phase == 1:
                    # the last accumulation into one of the rank's own chunks, its division for AVG
                    # and its quantization in two passes (:128-133, :155-162)
                    batch.setdefault(ops.SEG_REDUCE_DIV, []).append((r, c, ch, msg))
                elif msg is not None:
                    ops.dequantize_(ch, msg[0], msg[1], False)              # :204-209, nothing forwarded
                elif sending and (r, c) in own:
                    # the write-back of the rank's own codes (:167-172) and the quantization that
                    # forwards the chunk (:215), as one gather step
                    batch.setdefault(ops.SEG_GATHER, []).append((r, c, ch, own.pop((r, c))))
                elif sending:
                    batch.setdefault(ops.SEG_UNIFORM, []).append((r, c, ch, None))     # :138
            for kind, items in batch.items():
                chunks_k = [it[2] for it in items]
                if kind == ops.SEG_UNIFORM:
                    codes_k, luts_k = ops.uniform_8bit_quantize_segmented(chunks_k)
                else:
                    codes_k, luts_k = ops.ring_step_segmented(kind, chunks_k, [it[3][0] for it in items], [it[3][1] for it in items], div)
                for (r, c, _, _), codes, lut in zip(items, codes_k, luts_k):
                    if kind == ops.SEG_REDUCE_DIV:
                        own[(r, c)] = (codes, lut)
                    else:
                        posted.append(((r + 1) % W, step, codes, lut))
            for dst, st, codes, lut in posted:
                inbox[dst][st] = (codes, lut)
        if phase == 1 and W == 1:
            # one rank receives nothing: both chunks take the round trip on their own (:155-173)
            for i in range(BUFFER_COUNT):
                ch = chunk(0, i)
                if sources is not None:
                    codes, lut = touch(0, i, None, 1.0)
                else:
                    codes, lut = ops.uniform_8bit_quantize(ch, True)        # :162 (dividing by 1 changes nothing)
                if keep_codes:
                    final[0][i] = (codes, lut)
                else:
                    ops.dequantize_(ch, codes, lut, False)                  # :167-172
    assert not own
    return final if keep_codes else None


def ring_allreduce_single(tensor: torch.Tensor, avg: bool = False) -> None:
    """``ring_allreduce`` on a group of one rank: no message is sent, but both of the rank's
    chunks still take the lossy quantize / dequantize round trip (collectives.cpp:161-173).
    The two chunks are those of ``flat.chunk(2)`` (:90): ceil(n / 2) elements and the rest, so an
    odd number of elements is fine here, as it is in the reference's C++ (its Python twin's
    divisibility check, src/zeroband/collectives.py:83, only matters for more than one rank)."""
    flat = tensor.view(-1)
    n = flat.numel()
    if n % BUFFER_COUNT == 0:
        ring_allreduce_simulated([flat], avg=avg)
        return
    if n < BUFFER_COUNT:
        raise ValueError("a tensor of one element has no second chunk (collectives.cpp:161 indexes chunks[1])")
    _check_ring_inputs([flat[:n - 1]])          # dtype, contiguity
    first = (n + BUFFER_COUNT - 1) // BUFFER_COUNT
    for ch in (flat[:first], flat[first:]):
        codes, lut = ops.uniform_8bit_quantize(ch, True)                     # :162 (dividing by 1 changes nothing)
        ops.dequantize_(ch, codes, lut, False)                               # :167-172
