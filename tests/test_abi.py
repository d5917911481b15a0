"""The C-ABI library loads and exports what include/prime_hip.h declares (no GPU needed:
nothing here launches a kernel)."""
import ctypes
import re
from pathlib import Path

ROOT = Path(__file__).resolve().parents[1]
HEADER = ROOT / "include" / "prime_hip.h"


def declared_functions():
    text = HEADER.read_text()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(prime_[a-z0-9_]+)\s*\(", text)))


def test_header_and_binding_table_agree():
    from prime_amd import _lib

    assert declared_functions() == sorted(_lib.SIGNATURES)


def test_library_exports_every_declared_symbol():
    from prime_amd import _lib

    lib = _lib.load()
    for name in declared_functions():
        assert hasattr(lib, name), name
    assert lib.prime_hip_abi_version() == _lib.ABI_VERSION


def test_qparams_layout_matches_header():
    from prime_amd import _lib

    assert ctypes.sizeof(_lib.QParams) == 32
    assert _lib.QParams.scale.offset == 0 and _lib.QParams.inv_scale.offset == 4
    assert _lib.QParams.sum.offset == 8 and _lib.QParams.sumsq.offset == 16 and _lib.QParams.n.offset == 24


def test_argument_errors_are_reported_before_any_launch():
    from prime_amd import _lib

    lib = _lib.load()
    assert lib.prime_workspace_bytes() > 0
    assert lib.prime_quantize_u8(None, -1, 1.0, 128, None, None) == -1          # PRIME_EINVAL
    assert b"prime_quantize_u8" in lib.prime_hip_last_error()
    assert lib.prime_quantize_u8(None, 16, 1.0, 128, None, None) == -1          # null buffers with n > 0
    assert lib.prime_uniform_8bit_quantize(None, 0, None, None, None, None, None) == -1   # lut is required
    assert lib.prime_workspace_init(None, 0, None) == -2                          # PRIME_EWORKSPACE
    assert lib.prime_workspace_init(ctypes.c_void_p(4096), 16, None) == -2       # too small
    assert lib.prime_copy_bytes(ctypes.c_void_p(4096), ctypes.c_void_p(8192), 7, None) == -1
    assert lib.prime_average_buckets(ctypes.c_void_p(4096), ctypes.c_void_p(4096), 4, 0, ctypes.c_void_p(4096),
                                     None, ctypes.c_void_p(4096), None) == -1    # n_bins < 1
    p = ctypes.c_void_p(4096)
    assert lib.prime_uniform_8bit_quantize_batched(None, p, 3, p, p, None, None) == -1       # null x with tensors to do
    assert lib.prime_uniform_8bit_quantize_batched(p, p, 3, None, p, None, None) == -1       # null codes
    assert lib.prime_uniform_8bit_quantize_batched(p, None, 3, p, p, None, None) == -1       # null offsets
    assert lib.prime_uniform_8bit_quantize_batched(None, None, 0, None, None, None, None) == 0   # nothing to do
    assert lib.prime_ring_reduce_step(ctypes.c_void_p(4096), ctypes.c_void_p(4096), ctypes.c_void_p(4096), 4,
                                      ctypes.c_void_p(4096), ctypes.c_void_p(4096), None, None, None) == -2


def test_options_round_trip():
    from prime_amd import _lib

    old = _lib.get_option("blocks_per_cu")
    _lib.set_option("blocks_per_cu", 4)
    assert _lib.get_option("blocks_per_cu") == 4
    _lib.set_option("blocks_per_cu", old)
    try:
        _lib.set_option("no_such_option", 1)
    except _lib.PrimeHipError as e:
        assert "unknown option" in str(e)
    else:
        raise AssertionError("unknown option accepted")


def test_no_kernel_spills_and_streaming_kernels_keep_full_occupancy():
    # a spilled register in a bandwidth-bound kernel shows up as extra HBM traffic (scratch); the
    # streaming kernels are compiled for 8 wavefronts per SIMD, so two 1024-thread workgroups fit a CU
    from prime_amd.build import kernel_resources

    res = kernel_resources()
    assert len(res) >= 40
    spilled = {k: v["scratch"] for k, v in res.items() if v.get("scratch", 0) > 0}
    assert not spilled, spilled
    streaming = ("stats_kernel", "quantize_kernel", "hist_kernel", "dequant_kernel", "first_touch_kernel", "outer_step_kernel",
                 "pseudo_gradient_kernel", "div_kernel", "code_count_kernel", "code_remap_kernel", "copy_kernel")
    for name, v in res.items():
        if any(s in name for s in streaming):
            assert v["occupancy"] == 8 and v["vgprs"] <= 64, (name, v)


def test_built_in_scratch_is_a_dynamic_symbol_of_the_code_object():
    # the entry point that allocates nothing finds its scratch with hipGetSymbolAddress, which
    # resolves the name in the code object's dynamic symbols (and aborts when it is missing):
    # the array has to be exported there, at the size of one workspace
    from prime_amd import _lib
    from prime_amd.build import device_data_symbols

    syms = device_data_symbols()
    scratch = {k: v for k, v in syms.items() if "scratch" in k}
    assert len(scratch) == 1, syms
    (info,) = scratch.values()
    assert info["bind"] == "GLOBAL"
    assert info["size"] == _lib.load().prime_workspace_bytes()
