"""Direct calls into the C ABI for the GPU tests: torch supplies device memory and the
stream, every computation goes through libprime_hip.so entry points."""
from __future__ import annotations

import ctypes

import numpy as np
import torch

from prime_amd import _lib


class Abi:
    def __init__(self, dev: torch.device):
        self.dev = dev
        self.lib = _lib.load()
        self.st = torch.cuda.current_stream(dev).cuda_stream
        nbytes = int(self.lib.prime_workspace_bytes())
        self.ws = torch.empty(nbytes, dtype=torch.uint8, device=dev)
        _lib.check(self.lib.prime_workspace_init(self.ws.data_ptr(), nbytes, self.st), "workspace_init")

    def to_dev(self, a: np.ndarray) -> torch.Tensor:
        return torch.from_numpy(np.ascontiguousarray(a)).to(self.dev)

    def qparams(self, qp: torch.Tensor) -> dict:
        raw = qp.cpu().view(torch.uint8).numpy().tobytes()
        r = _lib.QParams.from_buffer_copy(raw[:32])
        return {"scale": np.float32(r.scale), "inv_scale": np.float32(r.inv_scale), "sum": r.sum, "sumsq": r.sumsq, "n": r.n}

    def uniform(self, x: torch.Tensor):
        n = x.numel()
        codes = torch.empty(n, dtype=torch.uint8, device=self.dev)
        lut = torch.empty(256, dtype=torch.float32, device=self.dev)
        qp = torch.empty(4, dtype=torch.float64, device=self.dev)
        _lib.check(self.lib.prime_uniform_8bit_quantize(x.data_ptr(), n, codes.data_ptr(), lut.data_ptr(), qp.data_ptr(),
                                                        self.ws.data_ptr(), self.st), "uniform")
        return codes, lut, qp

    def uniform_literal(self, x: torch.Tensor):
        n = x.numel()
        codes = torch.empty(n, dtype=torch.uint8, device=self.dev)
        lut = torch.empty(256, dtype=torch.float32, device=self.dev)
        qp = torch.empty(4, dtype=torch.float64, device=self.dev)
        _lib.check(self.lib.prime_uniform_8bit_quantize_literal(x.data_ptr(), n, codes.data_ptr(), lut.data_ptr(), qp.data_ptr(),
                                                                self.ws.data_ptr(), self.st), "uniform_literal")
        return codes, lut, qp

    def quantize_lookup(self, x: torch.Tensor, scale: float):
        n = x.numel()
        codes = torch.empty(n, dtype=torch.uint8, device=self.dev)
        lut = torch.empty(256, dtype=torch.float32, device=self.dev)
        _lib.check(self.lib.prime_quantize_lookup_u8(x.data_ptr(), n, ctypes.c_float(scale), codes.data_ptr(), lut.data_ptr(),
                                                     self.ws.data_ptr(), self.st), "quantize_lookup")
        return codes, lut

    def quantize(self, x: torch.Tensor, scale: float, zp: int = 128, codes: torch.Tensor | None = None):
        n = x.numel()
        if codes is None:
            codes = torch.empty(n, dtype=torch.uint8, device=self.dev)
        _lib.check(self.lib.prime_quantize_u8(x.data_ptr(), n, ctypes.c_float(scale), zp, codes.data_ptr(), self.st), "quantize")
        return codes

    def stats(self, x: torch.Tensor) -> dict:
        qp = torch.empty(4, dtype=torch.float64, device=self.dev)
        _lib.check(self.lib.prime_stats_f32(x.data_ptr(), x.numel(), qp.data_ptr(), self.ws.data_ptr(), self.st), "stats")
        return self.qparams(qp)

    def average_buckets(self, x: torch.Tensor, codes: torch.Tensor, n_bins: int = 256):
        lut = torch.empty(n_bins, dtype=torch.float32, device=self.dev)
        cnt = torch.zeros(256, dtype=torch.int64, device=self.dev)
        _lib.check(self.lib.prime_average_buckets(x.data_ptr(), codes.data_ptr(), x.numel(), n_bins, lut.data_ptr(),
                                                  cnt.data_ptr(), self.ws.data_ptr(), self.st), "average_buckets")
        return lut, cnt

    def dequant(self, out: torch.Tensor, lut: torch.Tensor, codes: torch.Tensor, add: bool):
        fn = self.lib.prime_dequant_add if add else self.lib.prime_dequant_set
        _lib.check(fn(out.data_ptr(), lut.data_ptr(), codes.data_ptr(), out.numel(), self.st), "dequant")

    def ring_step(self, acc: torch.Tensor, codes_in: torch.Tensor, lut_in: torch.Tensor, gather: bool = False,
                  divisor: float = None):
        n = acc.numel()
        codes = torch.empty(n, dtype=torch.uint8, device=self.dev)
        lut = torch.empty(256, dtype=torch.float32, device=self.dev)
        qp = torch.empty(4, dtype=torch.float64, device=self.dev)
        if divisor is not None:
            rc = self.lib.prime_ring_reduce_div_step(acc.data_ptr(), codes_in.data_ptr(), lut_in.data_ptr(), n, divisor,
                                                     codes.data_ptr(), lut.data_ptr(), qp.data_ptr(), self.ws.data_ptr(), self.st)
        else:
            fn = self.lib.prime_ring_gather_step if gather else self.lib.prime_ring_reduce_step
            rc = fn(acc.data_ptr(), codes_in.data_ptr(), lut_in.data_ptr(), n, codes.data_ptr(), lut.data_ptr(), qp.data_ptr(),
                    self.ws.data_ptr(), self.st)
        _lib.check(rc, "ring_step")
        return codes, lut, qp

    def requantize_codes(self, codes_in: torch.Tensor, lut_in: torch.Tensor, codes_out: torch.Tensor = None):
        n = codes_in.numel()
        codes = torch.empty(n, dtype=torch.uint8, device=self.dev) if codes_out is None else codes_out
        lut = torch.empty(256, dtype=torch.float32, device=self.dev)
        qp = torch.empty(4, dtype=torch.float64, device=self.dev)
        _lib.check(self.lib.prime_requantize_codes(codes_in.data_ptr(), lut_in.data_ptr(), n, codes.data_ptr(), lut.data_ptr(),
                                                   qp.data_ptr(), self.ws.data_ptr(), self.st), "requantize_codes")
        return codes, lut, qp

    def batched(self, flat: torch.Tensor, offsets: torch.Tensor):
        count = offsets.numel() - 1
        codes = torch.empty(flat.numel(), dtype=torch.uint8, device=self.dev)
        luts = torch.empty((count, 256), dtype=torch.float32, device=self.dev)
        qps = torch.empty((count, 4), dtype=torch.float64, device=self.dev)
        _lib.check(self.lib.prime_uniform_8bit_quantize_batched(flat.data_ptr(), offsets.data_ptr(), count, codes.data_ptr(),
                                                                luts.data_ptr(), qps.data_ptr(), self.st), "batched")
        return codes, luts, qps


def announce(msg: str) -> None:
    """Name the case before its GPU step, flushed, so a lost box still tells which one ran."""
    print(f"[gpu-case] {msg}", flush=True)


def _ptrs(tensors):
    return (ctypes.c_void_p * len(tensors))(*[t.data_ptr() for t in tensors])


def segmented_uniform(abi: Abi, xs):
    """prime_uniform_8bit_quantize_segmented on a list of device tensors."""
    count = len(xs)
    codes = [torch.empty(x.numel(), dtype=torch.uint8, device=abi.dev) for x in xs]
    luts = torch.empty((count, 256), dtype=torch.float32, device=abi.dev)
    qps = torch.empty((count, 4), dtype=torch.float64, device=abi.dev)
    ns = (ctypes.c_int64 * count)(*[x.numel() for x in xs])
    _lib.check(abi.lib.prime_uniform_8bit_quantize_segmented(_ptrs(xs), ns, count, _ptrs(codes), luts.data_ptr(), qps.data_ptr(),
                                                             abi.ws.data_ptr(), abi.st), "uniform_segmented")
    return codes, luts, qps


def segmented_ring_step(abi: Abi, kind: str, accs, codes_in, luts_in, divisor: float = 1.0):
    """prime_ring_{reduce,gather,reduce_div}_step_segmented on lists of device tensors (accs in place)."""
    count = len(accs)
    codes = [torch.empty(a.numel(), dtype=torch.uint8, device=abi.dev) for a in accs]
    luts = torch.empty((count, 256), dtype=torch.float32, device=abi.dev)
    qps = torch.empty((count, 4), dtype=torch.float64, device=abi.dev)
    ns = (ctypes.c_int64 * count)(*[a.numel() for a in accs])
    args = (_ptrs(accs), _ptrs(codes_in), _ptrs(luts_in), ns, count)
    tail = (_ptrs(codes), luts.data_ptr(), qps.data_ptr(), abi.ws.data_ptr(), abi.st)
    if kind == "reduce":
        rc = abi.lib.prime_ring_reduce_step_segmented(*args, *tail)
    elif kind == "gather":
        rc = abi.lib.prime_ring_gather_step_segmented(*args, *tail)
    else:
        rc = abi.lib.prime_ring_reduce_div_step_segmented(*args, ctypes.c_float(divisor), *tail)
    _lib.check(rc, f"ring_{kind}_step_segmented")
    return codes, luts, qps
