"""``torch.library`` registration of the compression ops over the C ABI.

Schemas mirror the Python signatures of the reference's wrappers
(src/zeroband/C/compression.py:11,22,34) plus the ops the ring needs
(src/zeroband/C/csrc/collectives.cpp:8-22,124-138):

    prime::uniform_8bit_quantize(Tensor tensor, bool inplace=True) -> (Tensor, Tensor)
    prime::average_buckets(Tensor tensor, Tensor quant_weight, int n_bins) -> Tensor
    prime::quantize_per_tensor_uint8(Tensor tensor, float scale, int zero_point) -> Tensor
    prime::dequantize(Tensor codes, Tensor lut) -> Tensor
    prime::dequantize_(Tensor(a!) out, Tensor codes, Tensor lut, bool accumulate) -> ()
    prime::ring_reduce_step(Tensor(a!) acc, Tensor codes_in, Tensor lut_in) -> (Tensor, Tensor)
    prime::ring_gather_step(Tensor(a!) chunk, Tensor codes_in, Tensor lut_in) -> (Tensor, Tensor)
    prime::requantize_codes(Tensor codes_in, Tensor lut_in) -> (Tensor, Tensor)
    prime::uniform_8bit_quantize_literal(Tensor tensor) -> (Tensor, Tensor)
    prime::ring_reduce_div_step(Tensor(a!) acc, Tensor codes_in, Tensor lut_in, float divisor) -> (Tensor, Tensor)
    prime::uniform_8bit_quantize_stats(Tensor tensor) -> (Tensor, Tensor, Tensor)
    prime::uniform_8bit_quantize_batched(Tensor flat, Tensor offsets) -> (Tensor, Tensor, Tensor)

Kernels exist for ROCm tensors only.  A CPU tensor reaches no kernel and the dispatcher
raises: there is deliberately no CPU path here.

torch is used for device memory (outputs come from its caching allocator) and for the
current stream; all arithmetic happens in libprime_hip.so.
"""
from __future__ import annotations

from typing import Dict, Optional, Tuple

import torch

from . import _lib

N_BINS = 256      # src/zeroband/C/csrc/compression.cpp:5
ZERO_POINT = 128  # compression.cpp:107

_LIB = torch.library.Library("prime", "DEF")
_LIB.define("uniform_8bit_quantize(Tensor tensor, bool inplace=True) -> (Tensor, Tensor)")
_LIB.define("average_buckets(Tensor tensor, Tensor quant_weight, int n_bins) -> Tensor")
_LIB.define("quantize_per_tensor_uint8(Tensor tensor, float scale, int zero_point) -> Tensor")
_LIB.define("dequantize(Tensor codes, Tensor lut) -> Tensor")
_LIB.define("dequantize_(Tensor(a!) out, Tensor codes, Tensor lut, bool accumulate) -> ()")
_LIB.define("ring_reduce_step(Tensor(a!) acc, Tensor codes_in, Tensor lut_in) -> (Tensor, Tensor)")
_LIB.define("ring_gather_step(Tensor(a!) chunk, Tensor codes_in, Tensor lut_in) -> (Tensor, Tensor)")
_LIB.define("uniform_8bit_quantize_literal(Tensor tensor) -> (Tensor, Tensor)")
_LIB.define("requantize_codes(Tensor codes_in, Tensor lut_in) -> (Tensor, Tensor)")
_LIB.define("ring_reduce_div_step(Tensor(a!) acc, Tensor codes_in, Tensor lut_in, float divisor) -> (Tensor, Tensor)")
_LIB.define("uniform_8bit_quantize_stats(Tensor tensor) -> (Tensor, Tensor, Tensor)")
_LIB.define("uniform_8bit_quantize_batched(Tensor flat, Tensor offsets) -> (Tensor, Tensor, Tensor)")

_workspaces: Dict[Tuple[int, int], torch.Tensor] = {}

_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _index(device: torch.device) -> int:
    return device.index if device.index is not None else torch.cuda.current_device()


def _stream(device: torch.device) -> int:
    """The current HIP stream of ``device`` as an integer handle."""
    if _raw_stream is not None:
        return _raw_stream(_index(device))
    return torch.cuda.current_stream(device).cuda_stream


class _NoGuard:
    def __enter__(self):
        return None

    def __exit__(self, *exc):
        return False


_NO_GUARD = _NoGuard()


def _on(device: torch.device):
    """Context that makes ``device`` current; free when it already is (the usual case)."""
    return _NO_GUARD if torch.cuda.current_device() == _index(device) else torch.cuda.device(device)


def workspace(device: torch.device, stream: Optional[int] = None) -> torch.Tensor:
    """The per-(device, stream) scratch block the multi-workgroup kernels share.  Work on one
    stream is ordered, so one block per stream is enough.  The key is the stream's handle: torch's own
    streams come from a pool and keep theirs for the life of the process; a caller that destroys an
    external stream with work in flight and creates another should call ``drop_workspaces()`` in between,
    since the new stream may be given the old handle and, with it, a block the old work still writes."""
    idx = _index(device)
    key = (idx, _stream(device) if stream is None else stream)
    ws = _workspaces.get(key)
    if ws is None:
        lib = _lib.load()
        nbytes = int(lib.prime_workspace_bytes())
        with torch.cuda.device(idx):
            ws = torch.empty(nbytes, dtype=torch.uint8, device=torch.device("cuda", idx))
            _lib.check(lib.prime_workspace_init(ws.data_ptr(), nbytes, key[1]), "prime_workspace_init")
        _workspaces[key] = ws
    return ws


def drop_workspaces() -> None:
    """Forget every cached workspace (after the device has been synchronised)."""
    _workspaces.clear()


def _need_f32(t: torch.Tensor, name: str) -> None:
    # the reference reads data_ptr<float>(): any other dtype is a c10::Error -> RuntimeError
    if t.dtype != torch.float32:
        raise RuntimeError(f"{name}: expected scalar type Float but found {t.dtype}")


def _need_u8(t: torch.Tensor, name: str) -> None:
    if t.dtype != torch.uint8:
        raise RuntimeError(f"{name}: expected scalar type Byte but found {t.dtype}")


def _need_lut(lut: torch.Tensor, name: str) -> torch.Tensor:
    _need_f32(lut, name)
    if lut.numel() < N_BINS:
        raise RuntimeError(f"{name}: lookup table needs {N_BINS} entries, got {lut.numel()}")
    return lut.contiguous()


def _uniform_8bit_quantize(tensor: torch.Tensor, inplace: bool = True):
    return _uniform_8bit_quantize_with(tensor, False, False)[:2]


def _uniform_8bit_quantize_literal(tensor: torch.Tensor):
    """uniform_8bit_quantize with the norm accumulated as libtorch's CPU kernel does it, so that
    scale and codes are the reference's bit for bit (compression.cpp:113); slow by design."""
    return _uniform_8bit_quantize_with(tensor, True, False)[:2]


def _uniform_8bit_quantize_stats(tensor: torch.Tensor):
    """(codes, lut, qparams): qparams is the 32-byte ``prime_qparams`` record as 4 float64
    words; view it with ``unpack_qparams``."""
    return _uniform_8bit_quantize_with(tensor, False, True)


def _uniform_8bit_quantize_with(tensor: torch.Tensor, literal: bool, want_qparams: bool):
    if tensor.dtype != torch.float32:
        _need_f32(tensor, "uniform_8bit_quantize")
    lib = _lib.load()
    x = tensor if tensor.is_contiguous() else tensor.contiguous()
    dev = x.device
    with _on(dev):
        st = _stream(dev)
        codes = torch.empty(x.shape, dtype=torch.uint8, device=dev)
        lut = torch.empty(N_BINS, dtype=torch.float32, device=dev)
        qp = torch.empty(4, dtype=torch.float64, device=dev) if want_qparams else None
        ws = workspace(dev, st)
        fn = lib.prime_uniform_8bit_quantize_literal if literal else lib.prime_uniform_8bit_quantize
        rc = fn(x.data_ptr(), x.numel(), codes.data_ptr(), lut.data_ptr(), qp.data_ptr() if want_qparams else None, ws.data_ptr(), st)
        if rc:
            _lib.check(rc, "prime_uniform_8bit_quantize")
    return codes, lut, qp


def uniform_8bit_quantize_out(tensor: torch.Tensor, codes: torch.Tensor, lut: torch.Tensor,
                              qparams: Optional[torch.Tensor] = None) -> None:
    """``uniform_8bit_quantize`` into buffers the caller keeps (a ring's send slots, a bucket's
    persistent code buffer): no allocation, about 1.7 us of host time on top of the three launches.
    ``codes`` uint8 with the tensor's number of elements, ``lut`` float32[256], ``qparams`` (optional)
    4 float64 words; all contiguous, on the tensor's device."""
    if tensor.dtype != torch.float32 or codes.dtype != torch.uint8 or lut.dtype != torch.float32:
        raise RuntimeError("uniform_8bit_quantize_out: expected a Float tensor, Byte codes and a Float lookup table")
    if codes.numel() != tensor.numel() or lut.numel() < N_BINS or (qparams is not None and qparams.numel() * qparams.element_size() < 32):
        raise RuntimeError("uniform_8bit_quantize_out: codes need the tensor's numel, lut 256 entries, qparams 32 bytes")
    if not (tensor.is_contiguous() and codes.is_contiguous() and lut.is_contiguous()):
        raise RuntimeError("uniform_8bit_quantize_out: tensor, codes and lut must be contiguous")
    if not tensor.is_cuda or codes.device != tensor.device or lut.device != tensor.device:
        raise RuntimeError("uniform_8bit_quantize_out: tensor, codes and lut must live on one ROCm device")
    lib = _lib.load()
    dev = tensor.device
    with _on(dev):
        st = _stream(dev)
        rc = lib.prime_uniform_8bit_quantize(tensor.data_ptr(), tensor.numel(), codes.data_ptr(), lut.data_ptr(),
                                             qparams.data_ptr() if qparams is not None else None, workspace(dev, st).data_ptr(), st)
        if rc:
            _lib.check(rc, "prime_uniform_8bit_quantize")


def _average_buckets(tensor: torch.Tensor, quant_weight: torch.Tensor, n_bins: int) -> torch.Tensor:
    _need_f32(tensor, "average_buckets")
    _need_u8(quant_weight, "average_buckets")
    if tensor.numel() != quant_weight.numel():
        raise RuntimeError("average_buckets: tensor and quant_weight differ in numel")
    lib = _lib.load()
    x = tensor.contiguous()
    q = quant_weight.contiguous()
    dev = x.device
    with _on(dev):
        lut = torch.empty(int(n_bins), dtype=torch.float32, device=dev)
        st = _stream(dev)
        ws = workspace(dev, st)
        _lib.check(
            lib.prime_average_buckets(x.data_ptr(), q.data_ptr(), x.numel(), int(n_bins), lut.data_ptr(), None,
                                      ws.data_ptr(), st),
            "prime_average_buckets")
    return lut


def _quantize_per_tensor_uint8(tensor: torch.Tensor, scale: float, zero_point: int) -> torch.Tensor:
    _need_f32(tensor, "quantize_per_tensor_uint8")
    lib = _lib.load()
    x = tensor.contiguous()
    dev = x.device
    with _on(dev):
        codes = torch.empty(x.shape, dtype=torch.uint8, device=dev)
        _lib.check(
            lib.prime_quantize_u8(x.data_ptr(), x.numel(), float(scale), int(zero_point), codes.data_ptr(), _stream(dev)),
            "prime_quantize_u8")
    return codes


def _dequantize(codes: torch.Tensor, lut: torch.Tensor) -> torch.Tensor:
    _need_u8(codes, "dequantize")
    out = torch.empty(codes.shape, dtype=torch.float32, device=codes.device)
    _dequantize_(out, codes, lut, False)
    return out


def _dequantize_(out: torch.Tensor, codes: torch.Tensor, lut: torch.Tensor, accumulate: bool) -> None:
    _need_f32(out, "dequantize_")
    _need_u8(codes, "dequantize_")
    lut = _need_lut(lut, "dequantize_")
    if not out.is_contiguous():
        raise RuntimeError("dequantize_: out must be contiguous (it is written in place)")
    if out.numel() != codes.numel():
        raise RuntimeError("dequantize_: out and codes differ in numel")
    lib = _lib.load()
    c = codes.contiguous()
    dev = out.device
    with _on(dev):
        fn = lib.prime_dequant_add if accumulate else lib.prime_dequant_set
        _lib.check(fn(out.data_ptr(), lut.data_ptr(), c.data_ptr(), out.numel(), _stream(dev)), "prime_dequant")


def _ring_reduce_step(acc: torch.Tensor, codes_in: torch.Tensor, lut_in: torch.Tensor):
    return _ring_step(acc, codes_in, lut_in, "ring_reduce_step")


def _ring_gather_step(chunk: torch.Tensor, codes_in: torch.Tensor, lut_in: torch.Tensor):
    return _ring_step(chunk, codes_in, lut_in, "ring_gather_step")


def _requantize_codes(codes_in: torch.Tensor, lut_in: torch.Tensor):
    """uniform_8bit_quantize(lut_in[codes_in]) computed from the codes alone: what the all-gather
    forwards (collectives.cpp:204-215) when the fp32 chunk is not needed yet."""
    _need_u8(codes_in, "requantize_codes")
    lut_in = _need_lut(lut_in, "requantize_codes")
    lib = _lib.load()
    c = codes_in.contiguous()
    dev = c.device
    with _on(dev):
        codes = torch.empty(c.shape, dtype=torch.uint8, device=dev)
        lut = torch.empty(N_BINS, dtype=torch.float32, device=dev)
        st = _stream(dev)
        ws = workspace(dev, st)
        _lib.check(lib.prime_requantize_codes(c.data_ptr(), lut_in.data_ptr(), c.numel(), codes.data_ptr(), lut.data_ptr(), None,
                                              ws.data_ptr(), st), "prime_requantize_codes")
    return codes, lut


def _ring_reduce_div_step(acc: torch.Tensor, codes_in: torch.Tensor, lut_in: torch.Tensor, divisor: float):
    """acc = (acc + lut_in[codes_in]) / divisor, then its quantization: the last accumulation into
    a rank's own chunk with ReduceOp::AVG's division (collectives.cpp:124-133, :155-162)."""
    return _ring_step(acc, codes_in, lut_in, "ring_reduce_div_step", float(divisor))


def _ring_step(acc: torch.Tensor, codes_in: torch.Tensor, lut_in: torch.Tensor, which: str, divisor: float = None):
    _need_f32(acc, which)
    _need_u8(codes_in, which)
    lut_in = _need_lut(lut_in, which)
    if not acc.is_contiguous():
        raise RuntimeError(f"{which}: the chunk must be contiguous (it is updated in place)")
    if acc.numel() != codes_in.numel():
        raise RuntimeError(f"{which}: chunk and codes_in differ in numel")
    lib = _lib.load()
    c = codes_in.contiguous()
    dev = acc.device
    with _on(dev):
        codes = torch.empty(acc.shape, dtype=torch.uint8, device=dev)
        lut = torch.empty(N_BINS, dtype=torch.float32, device=dev)
        st = _stream(dev)
        ws = workspace(dev, st)
        if divisor is not None:
            rc = lib.prime_ring_reduce_div_step(acc.data_ptr(), c.data_ptr(), lut_in.data_ptr(), acc.numel(), divisor,
                                                codes.data_ptr(), lut.data_ptr(), None, ws.data_ptr(), st)
        else:
            fn = lib.prime_ring_reduce_step if which == "ring_reduce_step" else lib.prime_ring_gather_step
            rc = fn(acc.data_ptr(), c.data_ptr(), lut_in.data_ptr(), acc.numel(), codes.data_ptr(), lut.data_ptr(), None,
                    ws.data_ptr(), st)
        _lib.check(rc, f"prime_{which}")
    return codes, lut


BATCHED_MAX_ELEMS = 1 << 16      # the one-workgroup-per-tensor kernel is meant for tensors up to this size


def _uniform_8bit_quantize_batched(flat: torch.Tensor, offsets: torch.Tensor):
    """Every slice flat[offsets[t]:offsets[t+1]] quantized on its own, one launch.
    Returns (codes like flat, luts [count, 256], qparams [count, 4] float64 words).
    With ``offsets`` in host memory the sizes are checked, and a set that holds an entry of more than
    65,536 elements is routed through the segmented call; offsets that live on the device are read by
    the kernel alone and every entry gets one workgroup whatever its size."""
    _need_f32(flat, "uniform_8bit_quantize_batched")
    if offsets.dtype != torch.int64 or offsets.dim() != 1 or offsets.numel() < 1:
        raise RuntimeError("uniform_8bit_quantize_batched: offsets must be a 1-D int64 tensor of count+1 entries")
    if not flat.is_contiguous():
        raise RuntimeError("uniform_8bit_quantize_batched: flat must be contiguous")
    if not offsets.is_cuda:
        # offsets the host can see: checked, and a set with an entry too large for one workgroup (the batched
        # kernel gives every tensor exactly one) goes through the segmented call, which sizes the grid per tensor
        host = offsets.tolist()
        if host[0] < 0 or host[-1] > flat.numel() or any(b < a for a, b in zip(host, host[1:])):
            raise RuntimeError("uniform_8bit_quantize_batched: offsets must be non-decreasing and lie inside flat")
        if any(b - a > BATCHED_MAX_ELEMS for a, b in zip(host, host[1:])):
            views = [flat.view(-1)[a:b] for a, b in zip(host, host[1:])]
            codes = torch.empty(flat.shape, dtype=torch.uint8, device=flat.device)
            cviews = [codes.view(-1)[a:b] for a, b in zip(host, host[1:])]
            luts = torch.empty((len(views), N_BINS), dtype=torch.float32, device=flat.device)
            qps = torch.empty((len(views), 4), dtype=torch.float64, device=flat.device)
            if views:
                SegmentPlan(SEG_UNIFORM, views, codes=cviews, luts=luts, qparams=qps).run()
            return codes, luts, qps
    lib = _lib.load()
    dev = flat.device
    count = offsets.numel() - 1
    off = offsets.to(dev).contiguous()
    with _on(dev):
        codes = torch.empty(flat.shape, dtype=torch.uint8, device=dev)
        luts = torch.empty((count, N_BINS), dtype=torch.float32, device=dev)
        qps = torch.empty((count, 4), dtype=torch.float64, device=dev)
        _lib.check(
            lib.prime_uniform_8bit_quantize_batched(flat.data_ptr(), off.data_ptr(), count, codes.data_ptr(),
                                                    luts.data_ptr(), qps.data_ptr(), _stream(dev)),
            "prime_uniform_8bit_quantize_batched")
    return codes, luts, qps


_LIB.impl("uniform_8bit_quantize", _uniform_8bit_quantize, "CUDA")
_LIB.impl("average_buckets", _average_buckets, "CUDA")
_LIB.impl("quantize_per_tensor_uint8", _quantize_per_tensor_uint8, "CUDA")
_LIB.impl("dequantize", _dequantize, "CUDA")
_LIB.impl("dequantize_", _dequantize_, "CUDA")
_LIB.impl("ring_reduce_step", _ring_reduce_step, "CUDA")
_LIB.impl("ring_gather_step", _ring_gather_step, "CUDA")
_LIB.impl("uniform_8bit_quantize_literal", _uniform_8bit_quantize_literal, "CUDA")
_LIB.impl("requantize_codes", _requantize_codes, "CUDA")
_LIB.impl("ring_reduce_div_step", _ring_reduce_div_step, "CUDA")
_LIB.impl("uniform_8bit_quantize_stats", _uniform_8bit_quantize_stats, "CUDA")
_LIB.impl("uniform_8bit_quantize_batched", _uniform_8bit_quantize_batched, "CUDA")


# shape-only implementations so the ops can be traced
@torch.library.register_fake("prime::uniform_8bit_quantize")
def _(tensor, inplace=True):
    return tensor.new_empty(tensor.shape, dtype=torch.uint8), tensor.new_empty(N_BINS, dtype=torch.float32)


@torch.library.register_fake("prime::average_buckets")
def _(tensor, quant_weight, n_bins):
    return tensor.new_empty(n_bins, dtype=torch.float32)


@torch.library.register_fake("prime::quantize_per_tensor_uint8")
def _(tensor, scale, zero_point):
    return tensor.new_empty(tensor.shape, dtype=torch.uint8)


@torch.library.register_fake("prime::dequantize")
def _(codes, lut):
    return codes.new_empty(codes.shape, dtype=torch.float32)


@torch.library.register_fake("prime::ring_reduce_step")
def _(acc, codes_in, lut_in):
    return acc.new_empty(acc.shape, dtype=torch.uint8), acc.new_empty(N_BINS, dtype=torch.float32)


@torch.library.register_fake("prime::ring_gather_step")
def _(chunk, codes_in, lut_in):
    return chunk.new_empty(chunk.shape, dtype=torch.uint8), chunk.new_empty(N_BINS, dtype=torch.float32)


@torch.library.register_fake("prime::uniform_8bit_quantize_literal")
def _(tensor):
    return tensor.new_empty(tensor.shape, dtype=torch.uint8), tensor.new_empty(N_BINS, dtype=torch.float32)


@torch.library.register_fake("prime::requantize_codes")
def _(codes_in, lut_in):
    return codes_in.new_empty(codes_in.shape), codes_in.new_empty(N_BINS, dtype=torch.float32)


@torch.library.register_fake("prime::ring_reduce_div_step")
def _(acc, codes_in, lut_in, divisor):
    return acc.new_empty(acc.shape, dtype=torch.uint8), acc.new_empty(N_BINS, dtype=torch.float32)


@torch.library.register_fake("prime::dequantize_")
def _(out, codes, lut, accumulate):
    return None


@torch.library.register_fake("prime::uniform_8bit_quantize_stats")
def _(tensor):
    return (tensor.new_empty(tensor.shape, dtype=torch.uint8), tensor.new_empty(N_BINS, dtype=torch.float32),
            tensor.new_empty(4, dtype=torch.float64))


@torch.library.register_fake("prime::uniform_8bit_quantize_batched")
def _(flat, offsets):
    count = offsets.shape[0] - 1
    return (flat.new_empty(flat.shape, dtype=torch.uint8), flat.new_empty((count, N_BINS), dtype=torch.float32),
            flat.new_empty((count, 4), dtype=torch.float64))


def unpack_qparams(qp: torch.Tensor) -> dict:
    """Host view of one ``prime_qparams`` record (synchronises)."""
    raw = qp.detach().cpu().contiguous().view(torch.uint8).numpy().tobytes()
    rec = _lib.QParams.from_buffer_copy(raw[: _lib.QPARAMS_BYTES])
    return {"scale": rec.scale, "inv_scale": rec.inv_scale, "sum": rec.sum, "sumsq": rec.sumsq, "n": rec.n}


uniform_8bit_quantize = torch.ops.prime.uniform_8bit_quantize
average_buckets = torch.ops.prime.average_buckets
quantize_per_tensor_uint8 = torch.ops.prime.quantize_per_tensor_uint8
dequantize = torch.ops.prime.dequantize
dequantize_ = torch.ops.prime.dequantize_
ring_reduce_step = torch.ops.prime.ring_reduce_step
ring_gather_step = torch.ops.prime.ring_gather_step
ring_reduce_div_step = torch.ops.prime.ring_reduce_div_step
requantize_codes = torch.ops.prime.requantize_codes
uniform_8bit_quantize_literal = torch.ops.prime.uniform_8bit_quantize_literal
uniform_8bit_quantize_stats = torch.ops.prime.uniform_8bit_quantize_stats
uniform_8bit_quantize_batched = torch.ops.prime.uniform_8bit_quantize_batched


# --------------------------------------------------------------------------------------------
# The callers either side of the path (src/zeroband/diloco.py): pseudo-gradient and outer step.

_LIB.define("div_(Tensor(a!) x, float divisor) -> ()")
_LIB.define("pseudo_gradient_(Tensor(a!) out, Tensor outer, Tensor inner, float world_size) -> ()")
_LIB.define("ring_first_touch_(Tensor(a!) grad, Tensor outer, Tensor inner, float world_size, Tensor? codes_in, Tensor? lut_in, "
            "float divisor) -> (Tensor, Tensor)")
_LIB.define("outer_sgd_nesterov_(Tensor(a!) param, Tensor(b!) momentum_buf, Tensor grad, Tensor(c!)? inner, "
            "float lr, float momentum, bool first_step) -> ()")
_LIB.define("outer_sgd_nesterov_codes_(Tensor(a!) param, Tensor(b!) momentum_buf, Tensor codes, Tensor lut, "
            "Tensor(c!)? inner, float lr, float momentum, bool first_step) -> ()")


def _need_flat_f32(t: torch.Tensor, name: str, n: int) -> None:
    _need_f32(t, name)
    if not t.is_contiguous() or t.numel() != n:
        raise RuntimeError(f"{name}: operands must be contiguous fp32 tensors of one size")


def _div_(x: torch.Tensor, divisor: float) -> None:
    """chunk.div_(world_size) of the ring's AVG (collectives.cpp:155-159)."""
    _need_flat_f32(x, "div_", x.numel())
    dev = x.device
    with _on(dev):
        _lib.check(_lib.load().prime_div_f32(x.data_ptr(), x.numel(), float(divisor), _stream(dev)), "prime_div_f32")


def _pseudo_gradient_(out: torch.Tensor, outer: torch.Tensor, inner: torch.Tensor, world_size: float) -> None:
    n = out.numel()
    for t in (out, outer, inner):
        _need_flat_f32(t, "pseudo_gradient_", n)
    lib = _lib.load()
    dev = out.device
    with _on(dev):
        _lib.check(lib.prime_pseudo_gradient_f32(outer.data_ptr(), inner.data_ptr(), n, float(world_size), out.data_ptr(),
                                                 _stream(dev)), "prime_pseudo_gradient_f32")


def _ring_first_touch_(grad: torch.Tensor, outer: torch.Tensor, inner: torch.Tensor, world_size: float,
                       codes_in: Optional[torch.Tensor], lut_in: Optional[torch.Tensor], divisor: float):
    """A chunk's only visit in the reduce-scatter with the pseudo-gradient formed on the way:
    grad = (outer - inner) / world_size (diloco.py:93-101); with a received message
    grad = (grad + lut_in[codes_in]) / divisor (collectives.cpp:128-133, :155-159); then
    (codes, lut) = uniform_8bit_quantize(grad).  Returns (codes, lut)."""
    n = grad.numel()
    for t in (grad, outer, inner):
        _need_flat_f32(t, "ring_first_touch_", n)
    if (codes_in is None) != (lut_in is None):
        raise RuntimeError("ring_first_touch_: codes_in and lut_in go together")
    cp = lp = None
    if codes_in is not None:
        _need_u8(codes_in, "ring_first_touch_")
        lut_in = _need_lut(lut_in, "ring_first_touch_")
        if codes_in.numel() != n:
            raise RuntimeError("ring_first_touch_: chunk and codes_in differ in numel")
        codes_in = codes_in.contiguous()
        cp, lp = codes_in.data_ptr(), lut_in.data_ptr()
    lib = _lib.load()
    dev = grad.device
    with _on(dev):
        codes = torch.empty(grad.shape, dtype=torch.uint8, device=dev)
        lut = torch.empty(N_BINS, dtype=torch.float32, device=dev)
        st = _stream(dev)
        ws = workspace(dev, st)
        _lib.check(lib.prime_ring_first_touch(outer.data_ptr(), inner.data_ptr(), n, float(world_size), cp, lp, float(divisor),
                                              grad.data_ptr(), codes.data_ptr(), lut.data_ptr(), None, ws.data_ptr(), st),
                   "prime_ring_first_touch")
    return codes, lut


def _outer_sgd_nesterov_(param, momentum_buf, grad, inner, lr: float, momentum: float, first_step: bool) -> None:
    n = param.numel()
    for t in (param, momentum_buf, grad) + ((inner,) if inner is not None else ()):
        _need_flat_f32(t, "outer_sgd_nesterov_", n)
    lib = _lib.load()
    dev = param.device
    with _on(dev):
        _lib.check(lib.prime_outer_sgd_nesterov_f32(param.data_ptr(), momentum_buf.data_ptr(), grad.data_ptr(),
                                                    inner.data_ptr() if inner is not None else None, n, float(lr),
                                                    float(momentum), int(first_step), _stream(dev)),
                   "prime_outer_sgd_nesterov_f32")


def _outer_sgd_nesterov_codes_(param, momentum_buf, codes, lut, inner, lr: float, momentum: float, first_step: bool) -> None:
    n = param.numel()
    for t in (param, momentum_buf) + ((inner,) if inner is not None else ()):
        _need_flat_f32(t, "outer_sgd_nesterov_codes_", n)
    _need_u8(codes, "outer_sgd_nesterov_codes_")
    lut = _need_lut(lut, "outer_sgd_nesterov_codes_")
    if codes.numel() != n or not codes.is_contiguous():
        raise RuntimeError("outer_sgd_nesterov_codes_: codes must be contiguous and match param in numel")
    lib = _lib.load()
    dev = param.device
    with _on(dev):
        _lib.check(lib.prime_outer_sgd_nesterov_u8(param.data_ptr(), momentum_buf.data_ptr(), codes.data_ptr(), lut.data_ptr(),
                                                   inner.data_ptr() if inner is not None else None, n, float(lr),
                                                   float(momentum), int(first_step), _stream(dev)),
                   "prime_outer_sgd_nesterov_u8")


@torch.library.register_fake("prime::div_")
def _(x, divisor):
    return None


@torch.library.register_fake("prime::pseudo_gradient_")
def _(out, outer, inner, world_size):
    return None


@torch.library.register_fake("prime::ring_first_touch_")
def _(grad, outer, inner, world_size, codes_in, lut_in, divisor):
    return grad.new_empty(grad.shape, dtype=torch.uint8), grad.new_empty(N_BINS, dtype=torch.float32)


@torch.library.register_fake("prime::outer_sgd_nesterov_")
def _(param, momentum_buf, grad, inner, lr, momentum, first_step):
    return None


@torch.library.register_fake("prime::outer_sgd_nesterov_codes_")
def _(param, momentum_buf, codes, lut, inner, lr, momentum, first_step):
    return None


_LIB.impl("div_", _div_, "CUDA")
_LIB.impl("ring_first_touch_", _ring_first_touch_, "CUDA")
_LIB.impl("pseudo_gradient_", _pseudo_gradient_, "CUDA")
_LIB.impl("outer_sgd_nesterov_", _outer_sgd_nesterov_, "CUDA")
_LIB.impl("outer_sgd_nesterov_codes_", _outer_sgd_nesterov_codes_, "CUDA")
div_ = torch.ops.prime.div_
pseudo_gradient_ = torch.ops.prime.pseudo_gradient_
ring_first_touch_ = torch.ops.prime.ring_first_touch_
outer_sgd_nesterov_ = torch.ops.prime.outer_sgd_nesterov_
outer_sgd_nesterov_codes_ = torch.ops.prime.outer_sgd_nesterov_codes_


# --------------------------------------------------------------------------------------------
# Pipelined quantization of many large buckets (the per-layer loop of
# Diloco.sync_pseudo_gradient, src/zeroband/diloco.py:108-110, without the network in between).

PIPELINE_STREAMS = 2     # measured best on MI355X for 205 MB buckets (1: 6.14, 2: 6.46, 3: 6.34, 4: 6.23, 6: 6.28 TB/s)
_side_streams: Dict[int, list] = {}


def _pipeline_streams(dev: torch.device, n: int) -> list:
    idx = dev.index if dev.index is not None else torch.cuda.current_device()
    pool = _side_streams.setdefault(idx, [])
    while len(pool) < n:
        pool.append(torch.cuda.Stream(device=dev))     # default priority
    return pool[:n]


class BucketPlan:
    """Pointer tables for one set of buckets and their outputs, built once and replayed: the
    C entry point takes host arrays, and rebuilding them per call would cost more than the
    launches for small sets."""

    def __init__(self, tensors, codes, luts: torch.Tensor, qparams: torch.Tensor, n_streams: int = PIPELINE_STREAMS):
        import ctypes

        if len(tensors) != len(codes) or luts.shape != (len(tensors), N_BINS) or qparams.shape != (len(tensors), 4):
            raise RuntimeError("BucketPlan: outputs do not match the buckets")
        dev = luts.device
        for t, c in zip(tensors, codes):
            _need_f32(t, "quantize_buckets")
            _need_u8(c, "quantize_buckets")
            if not (t.is_contiguous() and c.is_contiguous()) or t.numel() != c.numel() or t.device != dev or c.device != dev:
                raise RuntimeError("quantize_buckets: buckets and codes must be contiguous, of equal size, on one device")
        if luts.dtype != torch.float32 or qparams.dtype != torch.float64 or not luts.is_contiguous() or not qparams.is_contiguous():
            raise RuntimeError("quantize_buckets: luts must be contiguous float32, qparams contiguous float64")
        self.keep = (list(tensors), list(codes), luts, qparams)      # the tables hold raw pointers
        self.dev = dev
        self.count = len(tensors)
        self.n_streams = max(1, min(int(n_streams), max(self.count, 1)))
        self.streams = _pipeline_streams(dev, self.n_streams)
        n = self.count
        self.xs = (ctypes.c_void_p * n)(*[t.data_ptr() for t in tensors])
        self.ns = (ctypes.c_int64 * n)(*[t.numel() for t in tensors])
        self.cs = (ctypes.c_void_p * n)(*[c.data_ptr() for c in codes])
        with _on(dev):
            self.ws = []
            for s in self.streams:
                with torch.cuda.stream(s):
                    self.ws.append(workspace(dev))
        self.wss = (ctypes.c_void_p * self.n_streams)(*[w.data_ptr() for w in self.ws])
        self.sts = (ctypes.c_void_p * self.n_streams)(*[s.cuda_stream for s in self.streams])

    def run(self) -> None:
        """Enqueue every bucket; returns with the current stream ordered after all of them."""
        lib = _lib.load()
        cur = torch.cuda.current_stream(self.dev)
        start = cur.record_event()
        for s in self.streams:
            s.wait_event(start)
        with torch.cuda.device(self.dev):
            _lib.check(
                lib.prime_uniform_8bit_quantize_buckets(self.xs, self.ns, self.count, self.cs, self.keep[2].data_ptr(),
                                                        self.keep[3].data_ptr(), self.wss, self.sts, self.n_streams),
                "prime_uniform_8bit_quantize_buckets")
        for s in self.streams:
            cur.wait_event(s.record_event())


def quantize_buckets(tensors, n_streams: int = PIPELINE_STREAMS):
    """uniform_8bit_quantize of every bucket in ``tensors``, spread over ``n_streams`` HIP streams so
    that one bucket's statistics pass overlaps its neighbours' quantize pass.  Results are those of
    calling uniform_8bit_quantize bucket by bucket.  Returns (list of codes, luts [count, 256],
    qparams [count, 4]); the current stream is ordered after all the work."""
    if len(tensors) == 0:
        raise RuntimeError("quantize_buckets: no buckets")
    dev = tensors[0].device
    xs = [t.contiguous() for t in tensors]
    with _on(dev):
        codes = [torch.empty(t.shape, dtype=torch.uint8, device=dev) for t in xs]
        luts = torch.empty((len(xs), N_BINS), dtype=torch.float32, device=dev)
        qps = torch.empty((len(xs), 4), dtype=torch.float64, device=dev)
    BucketPlan(xs, codes, luts, qps, n_streams).run()
    return codes, luts, qps


# --------------------------------------------------------------------------------------------
# Segmented launches: many mid-size tensors (the 2 * world_size chunks the ring cuts a layer
# bucket into, collectives.cpp:89-90; the chunks all simulated ranks work on in one step) in
# three kernel launches in all instead of three per tensor.

SEG_UNIFORM, SEG_REDUCE, SEG_GATHER, SEG_REDUCE_DIV = "uniform", "reduce", "gather", "reduce_div"


class SegmentPlan:
    """Pointer tables of one segmented call, built once and replayed (``run``): ``tensors`` are the
    fp32 tensors (``uniform``) or the ring chunks that a step updates in place; ``codes_in`` /
    ``luts_in`` the received messages of a ring step.  Outputs: ``codes`` (one uint8 tensor per
    input, allocated here unless given), ``luts`` [count, 256] float32 and ``qparams`` [count, 4]
    float64 words.  Results equal the one-tensor ops' bit for bit."""

    def __init__(self, kind: str, tensors, codes_in=None, luts_in=None, divisor: float = 1.0, codes=None,
                 luts: Optional[torch.Tensor] = None, qparams: Optional[torch.Tensor] = None):
        import ctypes

        if kind not in (SEG_UNIFORM, SEG_REDUCE, SEG_GATHER, SEG_REDUCE_DIV):
            raise ValueError(f"unknown segmented operation {kind!r}")
        if len(tensors) == 0:
            raise RuntimeError("segmented call: no tensors")
        ring = kind != SEG_UNIFORM
        if ring and (codes_in is None or luts_in is None or len(codes_in) != len(tensors) or len(luts_in) != len(tensors)):
            raise RuntimeError("segmented ring step: one (codes_in, lut_in) message per chunk is needed")
        dev = tensors[0].device
        n = len(tensors)
        xs = []
        for t in tensors:
            _need_f32(t, "segmented call")
            if t.device != dev or not t.is_cuda:
                raise RuntimeError("segmented call: all tensors must live on one ROCm device")
            if ring and not t.is_contiguous():
                raise RuntimeError("segmented ring step: chunks must be contiguous (they are updated in place)")
            xs.append(t if t.is_contiguous() else t.contiguous())
        cin, lin = [], []
        if ring:
            for t, c, l in zip(xs, codes_in, luts_in):
                _need_u8(c, "segmented ring step")
                if c.numel() != t.numel():
                    raise RuntimeError("segmented ring step: chunk and codes_in differ in numel")
                cin.append(c.contiguous())
                lin.append(_need_lut(l, "segmented ring step"))
        with _on(dev):
            if codes is None:
                codes = [torch.empty(t.shape, dtype=torch.uint8, device=dev) for t in xs]
            if luts is None:
                luts = torch.empty((n, N_BINS), dtype=torch.float32, device=dev)
        for t, c in zip(xs, codes):
            _need_u8(c, "segmented call")
            if c.numel() != t.numel() or not c.is_contiguous() or c.device != dev:
                raise RuntimeError("segmented call: codes must be contiguous uint8 tensors of the inputs' sizes on their device")
        if luts.shape != (n, N_BINS) or luts.dtype != torch.float32 or not luts.is_contiguous() or luts.device != dev:
            raise RuntimeError("segmented call: luts must be a contiguous float32 [count, 256] tensor")
        if qparams is not None and (qparams.shape != (n, 4) or qparams.dtype != torch.float64 or not qparams.is_contiguous()):
            raise RuntimeError("segmented call: qparams must be a contiguous float64 [count, 4] tensor")
        self.kind, self.dev, self.count, self.divisor = kind, dev, n, float(divisor)
        self.codes, self.luts, self.qparams = list(codes), luts, qparams
        self.keep = (xs, cin, lin)                   # the tables hold raw pointers
        self.xs = (ctypes.c_void_p * n)(*[t.data_ptr() for t in xs])
        self.ns = (ctypes.c_int64 * n)(*[t.numel() for t in xs])
        self.cs = (ctypes.c_void_p * n)(*[c.data_ptr() for c in self.codes])
        self.ci = (ctypes.c_void_p * n)(*[c.data_ptr() for c in cin]) if ring else None
        self.li = (ctypes.c_void_p * n)(*[l.data_ptr() for l in lin]) if ring else None

    def run(self) -> None:
        lib = _lib.load()
        dev = self.dev
        with _on(dev):
            st = _stream(dev)
            ws = workspace(dev, st).data_ptr()
            qp = self.qparams.data_ptr() if self.qparams is not None else None
            lp = self.luts.data_ptr()
            if self.kind == SEG_UNIFORM:
                rc = lib.prime_uniform_8bit_quantize_segmented(self.xs, self.ns, self.count, self.cs, lp, qp, ws, st)
            elif self.kind == SEG_REDUCE:
                rc = lib.prime_ring_reduce_step_segmented(self.xs, self.ci, self.li, self.ns, self.count, self.cs, lp, qp, ws, st)
            elif self.kind == SEG_GATHER:
                rc = lib.prime_ring_gather_step_segmented(self.xs, self.ci, self.li, self.ns, self.count, self.cs, lp, qp, ws, st)
            else:
                rc = lib.prime_ring_reduce_div_step_segmented(self.xs, self.ci, self.li, self.ns, self.count, self.divisor, self.cs, lp,
                                                              qp, ws, st)
            if rc:
                _lib.check(rc, f"segmented {self.kind}")


def uniform_8bit_quantize_segmented(tensors, want_qparams: bool = False):
    """uniform_8bit_quantize of every tensor in ``tensors`` in three launches per 64 tensors.
    Returns (list of codes, luts [count, 256]) and, with ``want_qparams``, qparams [count, 4]."""
    qps = torch.empty((len(tensors), 4), dtype=torch.float64, device=tensors[0].device) if want_qparams and len(tensors) else None
    plan = SegmentPlan(SEG_UNIFORM, tensors, qparams=qps)
    plan.run()
    codes = [c.view(t.shape) for c, t in zip(plan.codes, tensors)]
    return (codes, plan.luts, qps) if want_qparams else (codes, plan.luts)


def ring_step_segmented(kind: str, chunks, codes_in, luts_in, divisor: float = 1.0):
    """ring_reduce_step / ring_gather_step / ring_reduce_div_step on every chunk of ``chunks`` (in
    place) with its received message, in three launches.  Returns (list of codes, luts [count, 256]);
    row i of luts goes with codes i."""
    plan = SegmentPlan(kind, chunks, codes_in, luts_in, divisor)
    plan.run()
    return plan.codes, plan.luts


def _ptr_table(tensors):
    import ctypes

    return (ctypes.c_void_p * len(tensors))(*[None if t is None else t.data_ptr() for t in tensors])


def pseudo_gradient_segmented_(outs, outers, inners, world_size: float) -> None:
    """``pseudo_gradient_`` for every parameter of a list in one launch per 64 tensors: the loop of
    src/zeroband/diloco.py:93-99 with both copies of the parameters on the device."""
    import ctypes

    if not (len(outs) == len(outers) == len(inners)):
        raise RuntimeError("pseudo_gradient_segmented_: the three lists differ in length")
    if not outs:
        return
    for o, a, b in zip(outs, outers, inners):
        n = o.numel()
        for t in (o, a, b):
            _need_flat_f32(t, "pseudo_gradient_segmented_", n)
    dev = outs[0].device
    ns = (ctypes.c_int64 * len(outs))(*[o.numel() for o in outs])
    with _on(dev):
        _lib.check(_lib.load().prime_pseudo_gradient_f32_segmented(_ptr_table(outers), _ptr_table(inners), ns, len(outs), float(world_size),
                                                                   _ptr_table(outs), _stream(dev)), "prime_pseudo_gradient_f32_segmented")


def outer_sgd_nesterov_segmented_(params, momentum_bufs, grads, inners, lr: float, momentum: float, first_step: bool) -> None:
    """``outer_sgd_nesterov_`` for every parameter of a list in one launch per 64 tensors
    (src/zeroband/diloco.py:212-215, :137-144).  ``inners`` may be None or hold None entries."""
    import ctypes

    if not (len(params) == len(momentum_bufs) == len(grads)) or (inners is not None and len(inners) != len(params)):
        raise RuntimeError("outer_sgd_nesterov_segmented_: the lists differ in length")
    if not params:
        return
    for i, (p, m, g) in enumerate(zip(params, momentum_bufs, grads)):
        n = p.numel()
        for t in (p, m, g) + ((inners[i],) if inners is not None and inners[i] is not None else ()):
            _need_flat_f32(t, "outer_sgd_nesterov_segmented_", n)
    dev = params[0].device
    ns = (ctypes.c_int64 * len(params))(*[p.numel() for p in params])
    with _on(dev):
        _lib.check(_lib.load().prime_outer_sgd_nesterov_f32_segmented(_ptr_table(params), _ptr_table(momentum_bufs), _ptr_table(grads),
                                                                      _ptr_table(inners) if inners is not None else None, ns, len(params),
                                                                      float(lr), float(momentum), int(first_step), _stream(dev)),
                   "prime_outer_sgd_nesterov_f32_segmented")
