"""TEST INFRASTRUCTURE: numpy/ctypes face of the CPU oracle (``prime_oracle.cpp``).

The arithmetic lives in C++ (``liboracle.so``); this module only marshals numpy arrays,
restates the ring schedule of ``ring_allreduce`` for W simulated ranks in one process,
and loads the compiled reference (``oracle/_ref/compression.so``) when it has been built.

Reference lines followed:
  src/zeroband/C/csrc/compression.cpp:9-125     (through liboracle.so)
  src/zeroband/C/csrc/collectives.cpp:76-230    ``ring_allreduce_sim`` below
  src/zeroband/collectives.py:53-192            the readable Python twin of the same schedule

``ring_allreduce_sim`` is pinned by the schedule's own algebra (every rank ends with the
same owner-quantized chunks, error bounded by the per-hop scales) and by the reference
test's inequality (tests/test_c/test_collectives.py:57); the compiled reference cannot
run it (collectives.cpp does not build without the gloo headers).
"""
from __future__ import annotations

import ctypes
import importlib.util
from pathlib import Path
from typing import List, Optional, Tuple

import numpy as np

HERE = Path(__file__).resolve().parent
_LIB_PATH = HERE / "liboracle.so"
_REF_PATH = HERE / "_ref" / "compression.so"

N_BINS = 256           # compression.cpp:5
ZERO_POINT = 128       # compression.cpp:107
BUFFER_COUNT = 2       # collectives.cpp:6

_lib = None
_ref = None

_f32p = ctypes.POINTER(ctypes.c_float)
_u8p = ctypes.POINTER(ctypes.c_uint8)
_i64p = ctypes.POINTER(ctypes.c_int64)
_f64p = ctypes.POINTER(ctypes.c_double)


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not _LIB_PATH.exists():
            raise RuntimeError(f"{_LIB_PATH} missing: run `python oracle/build.py`")
        L = ctypes.CDLL(str(_LIB_PATH))
        L.oracle_hardware_threads.restype = ctypes.c_int
        L.oracle_quantize_per_tensor.argtypes = [_f32p, ctypes.c_int64, ctypes.c_float, ctypes.c_int32, ctypes.c_int, _u8p]
        L.oracle_average_buckets.argtypes = [_f32p, _u8p, ctypes.c_int64, ctypes.c_int64, ctypes.c_int, _f32p, _i64p]
        L.oracle_average_buckets_f64.argtypes = [_f32p, _u8p, ctypes.c_int64, ctypes.c_int64, _f64p, _i64p]
        L.oracle_norm_literal.argtypes = [_f32p, ctypes.c_int64]
        L.oracle_norm_literal.restype = ctypes.c_float
        L.oracle_stats_f64.argtypes = [_f32p, ctypes.c_int64, _f64p, _f64p]
        L.oracle_scale_from_norm.argtypes = [ctypes.c_float, ctypes.c_int64]
        L.oracle_scale_from_norm.restype = ctypes.c_float
        L.oracle_scale_exact.argtypes = [_f32p, ctypes.c_int64]
        L.oracle_scale_exact.restype = ctypes.c_float
        L.oracle_scale_literal.argtypes = [_f32p, ctypes.c_int64]
        L.oracle_scale_literal.restype = ctypes.c_float
        L.oracle_uniform_8bit_quantize.argtypes = [_f32p, ctypes.c_int64, ctypes.c_int, ctypes.c_int, _u8p, _f32p, _f32p]
        L.oracle_index_add.argtypes = [_f32p, _f32p, _u8p, ctypes.c_int64]
        L.oracle_index_set.argtypes = [_f32p, _f32p, _u8p, ctypes.c_int64]
        L.oracle_index_add_threads.argtypes = [_f32p, _f32p, _u8p, ctypes.c_int64, ctypes.c_int]
        L.oracle_index_set_threads.argtypes = [_f32p, _f32p, _u8p, ctypes.c_int64, ctypes.c_int]
        L.oracle_div_scalar.argtypes = [_f32p, ctypes.c_int64, ctypes.c_float]
        L.oracle_pseudo_gradient.argtypes = [_f32p, _f32p, ctypes.c_int64, ctypes.c_float, _f32p]
        L.oracle_outer_sgd_nesterov.argtypes = [_f32p, _f32p, _f32p, ctypes.c_int64, ctypes.c_float, ctypes.c_float, ctypes.c_int]
        _lib = L
    return _lib


def _f32(a: np.ndarray) -> np.ndarray:
    a = np.ascontiguousarray(a, dtype=np.float32)
    return a.reshape(-1)


def _p(a: np.ndarray, t):
    return a.ctypes.data_as(t)


def hardware_threads() -> int:
    return int(lib().oracle_hardware_threads())


def quantize_per_tensor_uint8(x: np.ndarray, scale: float, zero_point: int = ZERO_POINT, threads: int = 0) -> np.ndarray:
    """compression.cpp:9-43."""
    x = _f32(x)
    out = np.empty(x.size, np.uint8)
    lib().oracle_quantize_per_tensor(_p(x, _f32p), x.size, ctypes.c_float(scale), zero_point, threads, _p(out, _u8p))
    return out


def average_buckets(x: np.ndarray, codes: np.ndarray, n_bins: int = N_BINS, threads: int = 0,
                    return_counts: bool = False):
    """compression.cpp:45-104 (fp32 per-thread sums, merged in thread order)."""
    x = _f32(x)
    codes = np.ascontiguousarray(codes, dtype=np.uint8).reshape(-1)
    assert codes.size == x.size
    lut = np.zeros(n_bins, np.float32)
    cnt = np.zeros(n_bins, np.int64)
    lib().oracle_average_buckets(_p(x, _f32p), _p(codes, _u8p), x.size, n_bins, threads, _p(lut, _f32p), _p(cnt, _i64p))
    return (lut, cnt) if return_counts else lut


def average_buckets_f64(x: np.ndarray, codes: np.ndarray, n_bins: int = N_BINS) -> Tuple[np.ndarray, np.ndarray]:
    """Exact counts and fp64 means: the tolerance target for lookup tables."""
    x = _f32(x)
    codes = np.ascontiguousarray(codes, dtype=np.uint8).reshape(-1)
    mean = np.zeros(n_bins, np.float64)
    cnt = np.zeros(n_bins, np.int64)
    lib().oracle_average_buckets_f64(_p(x, _f32p), _p(codes, _u8p), x.size, n_bins, _p(mean, _f64p), _p(cnt, _i64p))
    return mean, cnt


def norm_literal(x: np.ndarray) -> np.float32:
    x = _f32(x)
    return np.float32(lib().oracle_norm_literal(_p(x, _f32p), x.size))


def stats_f64(x: np.ndarray) -> Tuple[float, float]:
    x = _f32(x)
    s = ctypes.c_double()
    q = ctypes.c_double()
    lib().oracle_stats_f64(_p(x, _f32p), x.size, ctypes.byref(s), ctypes.byref(q))
    return s.value, q.value


def scale_from_norm(norm: float, n: int) -> np.float32:
    return np.float32(lib().oracle_scale_from_norm(ctypes.c_float(norm), n))


def scale_exact(x: np.ndarray) -> np.float32:
    x = _f32(x)
    return np.float32(lib().oracle_scale_exact(_p(x, _f32p), x.size))


def scale_literal(x: np.ndarray) -> np.float32:
    x = _f32(x)
    return np.float32(lib().oracle_scale_literal(_p(x, _f32p), x.size))


def uniform_8bit_quantize(x: np.ndarray, norm: str = "exact", scale: Optional[float] = None,
                          threads: int = 0) -> Tuple[np.ndarray, np.ndarray, np.float32]:
    """compression.cpp:106-125.  norm = "literal" | "exact" | "given" (then pass scale)."""
    x = _f32(x)
    mode = {"literal": 0, "exact": 1, "given": 2}[norm]
    codes = np.empty(x.size, np.uint8)
    lut = np.zeros(N_BINS, np.float32)
    sc = ctypes.c_float(0.0 if scale is None else scale)
    lib().oracle_uniform_8bit_quantize(_p(x, _f32p), x.size, threads, mode, _p(codes, _u8p), _p(lut, _f32p), ctypes.byref(sc))
    return codes, lut, np.float32(sc.value)


def index_add(out: np.ndarray, lut: np.ndarray, codes: np.ndarray, threads: int = 1) -> None:
    """collectives.cpp:8-14 (in place).  threads=1 is the loop as shipped."""
    assert out.dtype == np.float32 and out.flags.c_contiguous and lut.dtype == np.float32 and codes.dtype == np.uint8
    if threads == 1:
        lib().oracle_index_add(_p(out, _f32p), _p(lut, _f32p), _p(codes, _u8p), out.size)
    else:
        lib().oracle_index_add_threads(_p(out, _f32p), _p(lut, _f32p), _p(codes, _u8p), out.size, threads)


def index_set(out: np.ndarray, lut: np.ndarray, codes: np.ndarray, threads: int = 1) -> None:
    """collectives.cpp:16-22 (in place)."""
    assert out.dtype == np.float32 and out.flags.c_contiguous and lut.dtype == np.float32 and codes.dtype == np.uint8
    if threads == 1:
        lib().oracle_index_set(_p(out, _f32p), _p(lut, _f32p), _p(codes, _u8p), out.size)
    else:
        lib().oracle_index_set_threads(_p(out, _f32p), _p(lut, _f32p), _p(codes, _u8p), out.size, threads)


def div_scalar(x: np.ndarray, d: float) -> None:
    assert x.dtype == np.float32 and x.flags.c_contiguous
    lib().oracle_div_scalar(_p(x, _f32p), x.size, ctypes.c_float(d))


def pseudo_gradient(outer: np.ndarray, inner: np.ndarray, world_size: float) -> np.ndarray:
    """src/zeroband/diloco.py:93-101: (outer - inner) / world_size in fp32."""
    outer, inner = _f32(outer), _f32(inner)
    out = np.empty(outer.size, np.float32)
    lib().oracle_pseudo_gradient(_p(outer, _f32p), _p(inner, _f32p), outer.size, ctypes.c_float(world_size), _p(out, _f32p))
    return out


def outer_sgd_nesterov(param: np.ndarray, buf: np.ndarray, grad: np.ndarray, lr: float, momentum: float, first_step: bool) -> None:
    """One step of torch.optim.SGD(lr, momentum, nesterov=True) (diloco.py:72-74), in place on
    param and buf."""
    assert param.dtype == np.float32 and buf.dtype == np.float32 and param.flags.c_contiguous and buf.flags.c_contiguous
    grad = _f32(grad)
    lib().oracle_outer_sgd_nesterov(_p(param, _f32p), _p(buf, _f32p), _p(grad, _f32p), param.size, ctypes.c_float(lr),
                                    ctypes.c_float(momentum), int(first_step))


def torch_chunk_bounds(n: int, parts: int) -> List[Tuple[int, int]]:
    """Boundaries ``torch.chunk(parts)`` gives a 1-D tensor of n elements (collectives.cpp:90):
    pieces of ceil(n / parts), the last one shorter, possibly fewer than ``parts`` pieces."""
    size = -(-n // parts) if n else 0
    if size == 0:
        return [(0, 0)]
    return [(lo, min(n, lo + size)) for lo in range(0, n, size)]


def ring_hops(chunks: List[np.ndarray], norm: str = "exact"):
    """Per-hop compute of the reduce-scatter phase along one chunk's path round the ring
    (collectives.cpp:115-152 seen from the chunk): chunks[0] is quantized; every later
    holder adds the dequantized codes into its own copy and requantizes the result.
    Returns the list of (codes, lut, scale) sent on each hop and the final accumulator."""
    sent = []
    codes, lut, sc = uniform_8bit_quantize(chunks[0], norm)
    sent.append((codes, lut, sc))
    acc = None
    for r in range(1, len(chunks)):
        acc = np.array(chunks[r], dtype=np.float32, copy=True)
        index_add(acc, lut, codes)
        codes, lut, sc = uniform_8bit_quantize(acc, norm)
        sent.append((codes, lut, sc))
    return sent, acc


def ring_allreduce_sim(tensors: List[np.ndarray], avg: bool = False, norm: str = "exact") -> None:
    """collectives.cpp:76-230 for W ranks simulated in one process, in place.

    Messages are kept in per-(receiver, step) slots; ranks are stepped in lock step, which
    is equivalent to the reference's asynchronous send/recv with waits at step + 2
    (BUFFER_COUNT = 2).  Chunks are those of ``flat.chunk(2 W)`` (:90): the last one is shorter
    when 2 W does not divide numel (the Python twin asserts divisibility,
    src/zeroband/collectives.py:83; the C++ does not); numel must yield all 2 W chunks."""
    W = len(tensors)
    nb = BUFFER_COUNT * W
    n = tensors[0].size
    bounds = torch_chunk_bounds(n, nb)
    assert len(bounds) == nb, "torch.chunk gives fewer than 2 W chunks"
    flats = [t.reshape(-1) for t in tensors]

    def chunk(r, c):
        return flats[r][bounds[c][0]:bounds[c][1]]

    for phase in (1, 2):
        inbox = [dict() for _ in range(W)]   # inbox[rank][step] = (codes, lut)
        for step in range(1, nb + 1):
            posted = []
            for r in range(W):
                if phase == 1:
                    c = (r * BUFFER_COUNT - step) % nb                     # :116
                else:
                    c = (r * BUFFER_COUNT + BUFFER_COUNT - step) % nb      # :192
                ch = chunk(r, c)
                if (step - BUFFER_COUNT) in inbox[r]:                      # work posted at step-2 (:118)
                    codes, lut = inbox[r].pop(step - BUFFER_COUNT)
                    if phase == 1:
                        index_add(ch, lut, codes)                          # :128-133
                    else:
                        index_set(ch, lut, codes)                          # :204-209
                if step <= (W - 1) * BUFFER_COUNT:                         # :136 / :212
                    codes, lut, _ = uniform_8bit_quantize(ch, norm)        # :138 / :215
                    posted.append(((r + 1) % W, step, codes, lut))         # :140-150
            for dst, st, codes, lut in posted:
                inbox[dst][st] = (codes, lut)
        if phase == 1:
            for r in range(W):
                for i in range(BUFFER_COUNT):
                    ch = chunk(r, i + r * BUFFER_COUNT)
                    if avg:
                        div_scalar(ch, float(W))                           # :155-159
                    codes, lut, _ = uniform_8bit_quantize(ch, norm)        # :162
                    index_set(ch, lut, codes)                              # :167-172


# --------------------------------------------------------------------------------------
# The compiled reference (oracle/_ref/compression.so): the reference's own compression.cpp.


def ref_available() -> bool:
    return _REF_PATH.exists()


def ref():
    """The pybind11 module ``compression`` the reference declares (compression.cpp:129)."""
    global _ref
    if _ref is None:
        if not _REF_PATH.exists():
            raise RuntimeError(f"{_REF_PATH} missing: run `python oracle/build.py` where the reference is present")
        import torch  # noqa: F401  libtorch must be loaded first

        spec = importlib.util.spec_from_file_location("compression", str(_REF_PATH))
        mod = importlib.util.module_from_spec(spec)
        spec.loader.exec_module(mod)
        _ref = mod
    return _ref
