"""Drop-in for ``zeroband.C.compression`` (src/zeroband/C/compression.py): the same three
functions with the same signatures, running HIP kernels on ROCm tensors.

The reference compiles its C++ at import; here importing loads the prebuilt
libprime_hip.so and fails if it is absent.
"""
from typing import Tuple

import torch

from .. import _lib, ops

_lib.load()

_NORM_MODE = "exact"


def set_norm_mode(mode: str) -> None:
    """How ``uniform_8bit_quantize`` obtains ``tensor.norm()`` (compression.cpp:113).

    ``"exact"`` (default): the fp64 sum of squares, rounded once, at full memory bandwidth.
    ``"libtorch"``: the fp32 value the reference actually receives from libtorch's CPU kernel
    (eight serial lanes; 7e-4 below the exact norm at 2^24 elements, 3.7 % at 2^28), so that
    scale and codes equal a CPU run of the reference bit for bit; the accumulation is serial by
    definition and runs at about 1.9 G elements/s."""
    global _NORM_MODE
    if mode not in ("exact", "libtorch"):
        raise ValueError("norm mode must be 'exact' or 'libtorch'")
    _NORM_MODE = mode


def get_norm_mode() -> str:
    return _NORM_MODE


def uniform_8bit_quantize(tensor: torch.Tensor, inplace: bool = True) -> Tuple[torch.Tensor, torch.Tensor]:
    """Quantize a tensor to 8-bit codes and build the 256-entry lookup table.

    As in the reference (src/zeroband/C/csrc/compression.cpp:106-125) ``inplace`` is accepted
    and ignored, the input is never modified, no mean is subtracted and the zero point is 128.

    Returns:
        (uint8 codes shaped like ``tensor``, float32 lookup table of 256 bin means)
    """
    if _NORM_MODE == "libtorch":
        return ops.uniform_8bit_quantize_literal(tensor)
    if type(tensor) is torch.Tensor and tensor.is_cuda:
        return ops._uniform_8bit_quantize(tensor, inplace)      # straight to the C ABI: the dispatcher costs a microsecond
    return ops.uniform_8bit_quantize(tensor, inplace)           # CPU, fake and traced tensors: the registered op decides


def average_buckets(tensor: torch.Tensor, quant_weight: torch.Tensor, n_bins: int) -> torch.Tensor:
    """Mean of ``tensor`` over each code value of ``quant_weight`` (0.0 for an empty bin);
    compression.cpp:45-104."""
    return ops.average_buckets(tensor, quant_weight, n_bins)


def quantize_per_tensor_uint8(tensor: torch.Tensor, scale: float, zero_point: int) -> torch.Tensor:
    """``clamp(round(x * (1 / scale)) + zero_point, 0, 255)`` with ties away from zero;
    compression.cpp:9-43."""
    return ops.quantize_per_tensor_uint8(tensor, scale, zero_point)
