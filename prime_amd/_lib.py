"""ctypes binding of libprime_hip.so (the C ABI declared in include/prime_hip.h).

There is no fallback: if the library has not been built, importing anything that needs it
raises.  Build it with ``python -m prime_amd.build`` (hipcc, gfx950).
"""
from __future__ import annotations

import ctypes
from pathlib import Path

LIB_PATH = Path(__file__).resolve().parent / "csrc" / "libprime_hip.so"

ABI_VERSION = 2


class QParams(ctypes.Structure):
    """struct prime_qparams."""

    _fields_ = [
        ("scale", ctypes.c_float),
        ("inv_scale", ctypes.c_float),
        ("sum", ctypes.c_double),
        ("sumsq", ctypes.c_double),
        ("n", ctypes.c_int64),
    ]


class KernelTime(ctypes.Structure):
    """struct prime_kernel_time."""

    _fields_ = [
        ("name", ctypes.c_char * 40),
        ("launches", ctypes.c_int64),
        ("total_ms", ctypes.c_double),
        ("algo_bytes", ctypes.c_double),
    ]


QPARAMS_BYTES = ctypes.sizeof(QParams)
assert QPARAMS_BYTES == 32

_vp = ctypes.c_void_p
_i64 = ctypes.c_int64
_i32 = ctypes.c_int32
_f32 = ctypes.c_float

# name -> (restype, argtypes); every symbol include/prime_hip.h declares
SIGNATURES = {
    "prime_hip_abi_version": (ctypes.c_int, []),
    "prime_hip_last_error": (ctypes.c_char_p, []),
    "prime_hip_set_option": (ctypes.c_int, [ctypes.c_char_p, ctypes.c_int]),
    "prime_hip_get_option": (ctypes.c_int, [ctypes.c_char_p, ctypes.POINTER(ctypes.c_int)]),
    "prime_hip_profile_begin": (ctypes.c_int, []),
    "prime_hip_profile_end": (ctypes.c_int, [ctypes.POINTER(KernelTime), ctypes.c_int, ctypes.POINTER(ctypes.c_int)]),
    "prime_workspace_bytes": (_i64, []),
    "prime_workspace_init": (ctypes.c_int, [_vp, _i64, _vp]),
    "prime_stats_f32": (ctypes.c_int, [_vp, _i64, _vp, _vp, _vp]),
    "prime_quantize_u8": (ctypes.c_int, [_vp, _i64, _f32, _i32, _vp, _vp]),
    "prime_average_buckets": (ctypes.c_int, [_vp, _vp, _i64, _i64, _vp, _vp, _vp, _vp]),
    "prime_quantize_lookup_u8": (ctypes.c_int, [_vp, _i64, _f32, _vp, _vp, _vp, _vp]),
    "prime_uniform_8bit_quantize": (ctypes.c_int, [_vp, _i64, _vp, _vp, _vp, _vp, _vp]),
    "prime_uniform_8bit_quantize_noalloc": (ctypes.c_int, [_vp, _i64, _vp, _vp, _vp, _vp]),
    "prime_uniform_8bit_quantize_buckets": (ctypes.c_int, [_vp, _vp, _i64, _vp, _vp, _vp, _vp, _vp, ctypes.c_int]),
    "prime_uniform_8bit_quantize_batched": (ctypes.c_int, [_vp, _vp, _i64, _vp, _vp, _vp, _vp]),
    "prime_dequant_set": (ctypes.c_int, [_vp, _vp, _vp, _i64, _vp]),
    "prime_dequant_add": (ctypes.c_int, [_vp, _vp, _vp, _i64, _vp]),
    "prime_norm_literal_f32": (ctypes.c_int, [_vp, _i64, _vp, _vp, _vp]),
    "prime_uniform_8bit_quantize_literal": (ctypes.c_int, [_vp, _i64, _vp, _vp, _vp, _vp, _vp]),
    "prime_requantize_codes": (ctypes.c_int, [_vp, _vp, _i64, _vp, _vp, _vp, _vp, _vp]),
    "prime_ring_reduce_step": (ctypes.c_int, [_vp, _vp, _vp, _i64, _vp, _vp, _vp, _vp, _vp]),
    "prime_ring_gather_step": (ctypes.c_int, [_vp, _vp, _vp, _i64, _vp, _vp, _vp, _vp, _vp]),
    "prime_ring_reduce_div_step": (ctypes.c_int, [_vp, _vp, _vp, _i64, _f32, _vp, _vp, _vp, _vp, _vp]),
    "prime_uniform_8bit_quantize_segmented": (ctypes.c_int, [_vp, _vp, _i64, _vp, _vp, _vp, _vp, _vp]),
    "prime_ring_reduce_step_segmented": (ctypes.c_int, [_vp, _vp, _vp, _vp, _i64, _vp, _vp, _vp, _vp, _vp]),
    "prime_ring_reduce_div_step_segmented": (ctypes.c_int, [_vp, _vp, _vp, _vp, _i64, _f32, _vp, _vp, _vp, _vp, _vp]),
    "prime_ring_gather_step_segmented": (ctypes.c_int, [_vp, _vp, _vp, _vp, _i64, _vp, _vp, _vp, _vp, _vp]),
    "prime_div_f32": (ctypes.c_int, [_vp, _i64, _f32, _vp]),
    "prime_pseudo_gradient_f32": (ctypes.c_int, [_vp, _vp, _i64, _f32, _vp, _vp]),
    "prime_ring_first_touch": (ctypes.c_int, [_vp, _vp, _i64, _f32, _vp, _vp, _f32, _vp, _vp, _vp, _vp, _vp, _vp]),
    "prime_outer_sgd_nesterov_f32": (ctypes.c_int, [_vp, _vp, _vp, _vp, _i64, _f32, _f32, ctypes.c_int, _vp]),
    "prime_outer_sgd_nesterov_u8": (ctypes.c_int, [_vp, _vp, _vp, _vp, _vp, _i64, _f32, _f32, ctypes.c_int, _vp]),
    "prime_pseudo_gradient_f32_segmented": (ctypes.c_int, [_vp, _vp, _vp, _i64, _f32, _vp, _vp]),
    "prime_outer_sgd_nesterov_f32_segmented": (ctypes.c_int, [_vp, _vp, _vp, _vp, _vp, _i64, _f32, _f32, ctypes.c_int, _vp]),
    "prime_copy_bytes": (ctypes.c_int, [_vp, _vp, _i64, _vp]),
}

_lib = None


class PrimeHipError(RuntimeError):
    pass


def load() -> ctypes.CDLL:
    """Load the shared library and bind every declared entry point."""
    global _lib
    if _lib is not None:
        return _lib
    if not LIB_PATH.exists():
        raise PrimeHipError(
            f"{LIB_PATH} is missing: the HIP library is not built (run `python -m prime_amd.build`). "
            "There is no CPU fallback for these ops."
        )
    # The library needs libamdhip64.so.7, and so does torch, which ships a copy of its own: the first
    # one loaded serves the whole process.  torch's other ROCm libraries only work with torch's copy, so
    # torch goes first (loading this library first, then torch, crashes at the first GPU call).
    import torch  # noqa: F401

    lib = ctypes.CDLL(str(LIB_PATH))
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)   # AttributeError if the library lacks a declared symbol
        fn.restype = res
        fn.argtypes = args
    got = lib.prime_hip_abi_version()
    if got != ABI_VERSION:
        raise PrimeHipError(f"libprime_hip.so ABI version {got}, expected {ABI_VERSION}")
    _lib = lib
    return lib


def check(rc: int, what: str) -> None:
    if rc != 0:
        msg = load().prime_hip_last_error()
        raise PrimeHipError(f"{what} failed (code {rc}): {msg.decode() if msg else ''}")


def set_option(name: str, value: int) -> None:
    check(load().prime_hip_set_option(name.encode(), int(value)), f"set_option({name})")


def get_option(name: str) -> int:
    v = ctypes.c_int()
    check(load().prime_hip_get_option(name.encode(), ctypes.byref(v)), f"get_option({name})")
    return v.value


def profile_begin() -> None:
    check(load().prime_hip_profile_begin(), "profile_begin")


def profile_end() -> dict:
    """{kernel name: {"launches", "total_ms", "algo_bytes"}} since profile_begin (synchronises)."""
    cap = 64
    buf = (KernelTime * cap)()
    n = ctypes.c_int()
    check(load().prime_hip_profile_end(buf, cap, ctypes.byref(n)), "profile_end")
    return {buf[i].name.decode(): {"launches": buf[i].launches, "total_ms": buf[i].total_ms,
                                   "algo_bytes": buf[i].algo_bytes} for i in range(min(n.value, cap))}
