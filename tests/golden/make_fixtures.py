"""Writes tests/golden/uniform8_reference.npz with the compiled reference (oracle/_ref).

Run in the build container, where the reference checkout is present:

    python oracle/build.py && python tests/golden/make_fixtures.py

The reference's own tests hold no vectors for this path (tests/test_c/test_compression.py only
prints timings), so the fixtures are outputs of the reference's compression.cpp itself,
compiled unchanged from where it lies.  The file stores seeds rather than inputs where the
input is a plain seeded draw; inputs that are not (edge cases) are stored in full.

Cases: N(0, 1e-3) tensors of n in {1, 2, 7, 255, 4096, 65536} (seed = n), a Student-t(3)*1e-4
tensor (heavy tails: populated clip bins), a tensor with 50 % exact zeros, a constant
tensor, and the quantize_per_tensor_uint8 vector of the reference test
(tests/test_c/test_compression.py:46-48: ones * 10, scale 0.01, zero point 128).
"""
from __future__ import annotations

import sys
from pathlib import Path

import numpy as np
import torch

ROOT = Path(__file__).resolve().parents[2]
sys.path.insert(0, str(ROOT))
from oracle import oracle as O  # noqa: E402

OUT = Path(__file__).resolve().parent / "uniform8_reference.npz"
OUT_LARGE = Path(__file__).resolve().parent / "uniform8_reference_large.json"

# Large cases are stored as digests: the scale bits, the SHA-256 of the codes and the code
# populations.  At these sizes libtorch's norm differs visibly from the exact one (config 1 of the
# benchmark is "normal:16777216"; 2^26 is the ring chunk of config 3 and 2^28 the size the throughput target is quoted on,
# where the norm is 5e-3 and 3.7e-2 low), so they pin the literal path where it matters.
LARGE_CASES = ["normal:1048583", "student:4194304", "normal:16777216", "normal:67108864", "normal:268435456"]


def case_input(name: str) -> np.ndarray:
    """Inputs are regenerated from this function in the tests: keep it deterministic."""
    kind, arg = name.split(":")
    n = int(arg)
    rng = np.random.default_rng(n)
    if kind == "normal":
        return (rng.standard_normal(n) * 1e-3).astype(np.float32)
    if kind == "student":
        return (rng.standard_t(3, n) * 1e-4).astype(np.float32)
    if kind == "halfzero":
        x = (rng.standard_normal(n) * 1e-3).astype(np.float32)
        x[rng.random(n) < 0.5] = 0.0
        return x
    if kind == "const":
        return np.full(n, 0.25, np.float32)
    raise ValueError(name)


CASES = ["normal:1", "normal:2", "normal:7", "normal:255", "normal:4096", "normal:65536",
         "student:20000", "halfzero:10000", "const:5000"]


def main() -> None:
    R = O.ref()
    out = {}
    for name in CASES:
        x = case_input(name)
        codes, lut = R.uniform_8bit_quantize(torch.from_numpy(x.copy()), True)
        codes = codes.numpy().copy()
        lut = lut.numpy().copy()
        norm = np.float32(torch.from_numpy(x).norm().item())
        scale = O.scale_from_norm(float(norm), x.size)
        # the literal scale must reproduce the reference's codes through the restatement
        oc = O.quantize_per_tensor_uint8(x, float(scale), 128)
        assert np.array_equal(oc, codes), name
        key = name.replace(":", "_")
        out[f"{key}/codes"] = codes
        out[f"{key}/lut"] = lut
        out[f"{key}/norm"] = np.array([norm], np.float32)
        out[f"{key}/scale"] = np.array([scale], np.float32)
    # quantize_per_tensor_uint8 on its own: reference test vector and a spread of scales
    x = case_input("normal:4096") * 1000.0
    for i, scale in enumerate([0.01, 0.1, 0.5, 1.0, 3.0]):
        q = R.quantize_per_tensor_uint8(torch.from_numpy(x.copy()), scale, 128).numpy().copy()
        out[f"qpt_{i}/scale"] = np.array([scale], np.float64)
        out[f"qpt_{i}/codes"] = q
    ones = R.quantize_per_tensor_uint8(torch.ones(1000) * 10, 0.01, 128).numpy().copy()
    out["qpt_ones/codes"] = ones
    # average_buckets with codes that are not derived from the values
    rng = np.random.default_rng(7)
    xa = (rng.standard_normal(30000) * 10).astype(np.float32)
    ca = rng.integers(0, 255, 30000).astype(np.uint8)          # as the reference test draws them (:68)
    la = R.average_buckets(torch.from_numpy(xa.copy()), torch.from_numpy(ca.copy()), 256).numpy().copy()
    out["avg/x"] = xa
    out["avg/codes"] = ca
    out["avg/lut"] = la
    np.savez_compressed(OUT, **out)
    print("wrote", OUT, OUT.stat().st_size, "bytes")
    import hashlib
    import json

    large = {}
    for name in LARGE_CASES:
        x = case_input(name)
        codes, lut = R.uniform_8bit_quantize(torch.from_numpy(x.copy()), True)
        codes = codes.numpy()
        norm = np.float32(torch.from_numpy(x).norm().item())
        scale = O.scale_from_norm(float(norm), x.size)
        assert np.array_equal(O.quantize_per_tensor_uint8(x, float(scale), 128), codes), name
        large[name] = {
            "n": int(x.size),
            "norm_bits": int(np.array([norm], np.float32).view(np.uint32)[0]),
            "scale_bits": int(np.array([scale], np.float32).view(np.uint32)[0]),
            "codes_sha256": hashlib.sha256(codes.tobytes()).hexdigest(),
            "counts": np.bincount(codes, minlength=256).tolist(),
            "lut": [float(v) for v in lut.numpy()],
            "input_sha256": hashlib.sha256(x.tobytes()).hexdigest(),
        }
    OUT_LARGE.write_text(json.dumps(large, indent=1))
    print("wrote", OUT_LARGE, OUT_LARGE.stat().st_size, "bytes")


if __name__ == "__main__":
    main()
