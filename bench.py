#!/usr/bin/env python3
"""Benchmark of the int8 pseudo-gradient compression path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--legs a,b,...]

One "step" is one pass of the hot path, uniform_8bit_quantize (statistics pass, then the fused
quantize + 256-bin lookup build), over one 2^28-element fp32 tensor N(0, 1e-3): the size the
target is quoted on, 1 GiB, four times the last-level cache: the statistics pass reads all of it from
HBM, the quantize pass all but the tensor's last 256 MiB, which the statistics pass leaves in that cache.  Three
such tensors (torch generator on the GPU, seeds 0..2) and three code buffers are resident before
the timed region and visited in rotation.

The single JSON line printed at the end carries
  value          algorithmic GB/s of uniform_8bit_quantize (9 bytes per element: x read twice, codes
                 written once): K calls back to back between two synchronisations
  ring_step_2p28 the ring reduce step (dequantize-add + requantize, 14 bytes per element) at the same size
  roofline       the dominant kernel (quantize + histogram, 5 bytes per element) inside those calls,
                 priced against the 8 TB/s HBM peak from per-launch HIP-event times; the same kernel on
                 the 205 MB buckets of configuration 2 is listed beside it, as run and with its input cold
  tensor_2p28    every operation of the path on 2^28-element tensors, one row each: statistics,
                 quantize (a2), average_buckets (a3), dequantize add / set (a4 / a5), the fused
                 quantize + lookup, uniform_8bit_quantize and the ring reduce step
  config_2_buckets  benchmark configuration 2: the 22 per-layer buckets of a 1B model (51,380,224 elements each,
                 Student-t(3) * 1e-4), quantized bucket by bucket on one stream and dealt over two; a
                 205 MB bucket stays in the 256 MB last-level cache between its two passes: cache-assisted
  ring_step      benchmark configuration 3: W = 8 chunks of 2^26 elements; quantize chunk 0, then 7 hops of
                 dequantize-add + requantize (14 bytes per element per hop)
  ring_chunks    the sizes the ring really runs at: a layer bucket cut into 2 W = 16 chunks (3,211,264
                 elements for configuration 2, 1,860,119 for configuration 4) and 64 tensors of 2^20 elements;
                 one chunk at a time against all W = 8 ranks' chunks of a step in one segmented call
  other_configs  benchmark configurations 1, 4 and 5 (round trip on 2^24 elements; 42 buckets of a 10B model's
                 shard with outliers, quantize + dequantize; 2,000 small tensors in one launch and the
                 edge tensors), each as algorithmic GB/s
  cpu_baseline   the reference's own compression.cpp (compiled into oracle/_ref) on this box's
                 host cores, on the same tensor the GPU leg starts with (copied to the host), a few
                 repetitions, with the same operations one by one

--legs runs a subset (t28, buckets, ring, chunks, outer, diloco, configs, staging): what a profiler run
of one workload uses, so that every kernel name in its trace belongs to one element count.
"""
from __future__ import annotations

import argparse
import json
import os
import statistics
import sys
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
sys.path.insert(0, str(ROOT))

HBM_PEAK_GBS = 8000.0           # MI355X HBM3E
BUCKET_ELEMS = 4 * 2048 * 2048 + 3 * 2048 * 5632    # 51,380,224
N_LAYERS = 22
RING_W = 8
RING_CHUNK = 1 << 26
N28 = 1 << 28
RING_CHUNK_CFG2 = BUCKET_ELEMS // 16     # a layer bucket cut into 2 * W chunks for W = 8 (collectives.cpp:89-90)
RING_CHUNK_CFG4 = 29_761_904 // 16       # 1,860,119: the same for a 10B model's shard bucket


def measured_traffic(profile: str, kernel_prefix: str, min_total_mb: float = 0.0):
    """HBM bytes one launch of a kernel moves, from the committed summary of the two rocprofv3 --pmc
    runs (FETCH_SIZE, then WRITE_SIZE, each scaled by what the same counter reads for the 1 GiB copy
    this program runs first): the total_MB column of the kernel's row in profiles/<profile>.  None
    when the file or the row is missing."""
    path = ROOT / "profiles" / profile
    if not path.exists():
        return None
    best = None
    for line in path.read_text().splitlines():
        if line.startswith(kernel_prefix):
            try:
                total = float(line.split()[-1])
            except ValueError:
                continue
            if total >= min_total_mb and (best is None or total > best):
                best = total
    return None if best is None else best * 1e6


def student_t3(n, device, seed, scale):
    """Student-t with 3 degrees of freedom: z / sqrt(chi2_3 / 3), seeded per bucket."""
    import torch

    g = torch.Generator(device=device).manual_seed(seed)
    z = torch.randn(n, device=device, generator=g)
    chi = torch.zeros(n, device=device)
    for _ in range(3):
        w = torch.randn(n, device=device, generator=g)
        chi.addcmul_(w, w)
    z.div_(chi.div_(3.0).sqrt_()).mul_(scale)
    return z


def kernel_table(prof: dict, event_overhead_us: float) -> dict:
    """Per-kernel average duration (event bracket minus the measured bracket overhead) and the
    algorithmic GB/s it implies."""
    out = {}
    for k, v in prof.items():
        raw = v["total_ms"] / v["launches"] * 1e3
        us = max(raw - event_overhead_us, 1e-3)
        out[k] = {"avg_us": round(us, 2), "avg_us_event_bracket": round(raw, 2),
                  "algo_GBps": round(v["algo_bytes"] / v["launches"] / (us * 1e-6) / 1e9, 1)}
    return out


def _median_time(fn, reps: int) -> float:
    fn()
    times = []
    for _ in range(reps):
        t0 = time.perf_counter()
        fn()
        times.append(time.perf_counter() - t0)
    return statistics.median(times)


def cpu_baseline(x, acc, ring_codes, ring_lut, what: str, reps: int) -> dict:
    """The reference's CPU ops on this host on the tensors the GPU leg works on (numpy arrays copied
    from the device): ``x`` for uniform_8bit_quantize and its parts, ``acc`` with the message
    (``ring_codes``, ``ring_lut``) for the ring hop.  kind "reference" when oracle/_ref is present
    (the reference's compression.cpp compiled unchanged), else the restatement ("port").  The ring's
    dequantize loops exist only as a restatement (collectives.cpp does not build without the gloo
    headers); as shipped they run on one thread."""
    import torch
    from oracle import oracle as O

    sample_elems, ring_elems = x.size, acc.size
    threads = O.hardware_threads()
    if O.ref_available():
        R = O.ref()
        xt = torch.from_numpy(x)
        uniform = lambda t: R.uniform_8bit_quantize(t, True)                      # noqa: E731
        codes_t, _ = uniform(xt)
        scale = float(O.scale_literal(x))
        parts = {
            "norm_ms": _median_time(lambda: xt.norm(), reps) * 1e3,                                    # compression.cpp:113
            "quantize_ms": _median_time(lambda: R.quantize_per_tensor_uint8(xt, scale, 128), reps) * 1e3,   # :119
            "average_buckets_ms": _median_time(lambda: R.average_buckets(xt, codes_t, 256), reps) * 1e3,    # :122
        }
        fn = lambda: uniform(xt)                                                  # noqa: E731
        kind = "reference"
    else:
        uniform = None
        codes = O.quantize_per_tensor_uint8(x, float(O.scale_literal(x)), 128)
        parts = {
            "norm_ms": _median_time(lambda: O.norm_literal(x), reps) * 1e3,
            "quantize_ms": _median_time(lambda: O.quantize_per_tensor_uint8(x, 2e-5, 128), reps) * 1e3,
            "average_buckets_ms": _median_time(lambda: O.average_buckets(x, codes), reps) * 1e3,
        }
        fn = lambda: O.uniform_8bit_quantize(x, "literal")      # noqa: E731
        kind = "port"
    t = _median_time(fn, reps)

    # ring hop: chunk += lut[codes] on one thread as shipped, then uniform_8bit_quantize(chunk)
    rc, rl = ring_codes, ring_lut
    t_add = _median_time(lambda: O.index_add(acc, rl, rc, 1), 3)
    t_add_threads = _median_time(lambda: O.index_add(acc, rl, rc, threads), 3)
    t_set = _median_time(lambda: O.index_set(acc, rl, rc, 1), 3)
    if uniform is not None:
        at = torch.from_numpy(acc)
        t_q = _median_time(lambda: uniform(at), 3)
    else:
        t_q = _median_time(lambda: O.uniform_8bit_quantize(acc, "literal"), 3)
    hop = t_add + t_q
    return {
        "value": round(9.0 * sample_elems / t / 1e9, 3),
        "unit": "GB/s",
        "cores": threads,
        "kind": kind,
        "sample": f"uniform_8bit_quantize on {what} ({sample_elems} elements, copied from the GPU), median of {reps} runs "
                  f"after one warm-up, {threads} threads (hardware_concurrency, as compression.cpp:7), "
                  f"{os.cpu_count()} logical CPUs visible",
        "elements_per_s": round(sample_elems / t, 1),
        "ms_per_call": round(t * 1e3, 3),
        "breakdown_ms": {k: round(v, 3) for k, v in parts.items()},
        # the same operations one by one, as GB/s of their algorithmic bytes (beside tensor_2p28.operations)
        "operations": {
            "stats (norm)": {"GBps": round(4.0 * sample_elems / parts["norm_ms"] / 1e6, 3), "threads": 1, "elements": sample_elems},
            "quantize_per_tensor_uint8 (a2)": {"GBps": round(5.0 * sample_elems / parts["quantize_ms"] / 1e6, 3), "threads": threads,
                                               "elements": sample_elems},
            "average_buckets (a3)": {"GBps": round(5.0 * sample_elems / parts["average_buckets_ms"] / 1e6, 3), "threads": threads,
                                     "elements": sample_elems},
            "index_add (a4)": {"GBps": round(9.0 * ring_elems / t_add / 1e9, 3), "threads": 1, "elements": ring_elems,
                               "note": "as shipped: the OpenMP pragma is inert without -fopenmp (src/zeroband/C/collectives.py:17)"},
            "index_set (a5)": {"GBps": round(5.0 * ring_elems / t_set / 1e9, 3), "threads": 1, "elements": ring_elems},
            "uniform_8bit_quantize (a1)": {"GBps": round(9.0 * sample_elems / t / 1e9, 3), "threads": threads, "elements": sample_elems},
            "ring reduce step (a4 + a1)": {"GBps": round(14.0 * ring_elems / hop / 1e9, 3), "threads": threads, "elements": ring_elems},
        },
        "ring_step": {
            "value": round(14.0 * ring_elems / hop / 1e9, 3),
            "unit": "GB/s",
            "kind": kind + " quantize + port index_add (1 thread, as shipped)",
            "sample": f"one hop on a {ring_elems}-element chunk (the first quarter of the GPU leg's accumulator and message), median of 3",
            "ms_per_hop": round(hop * 1e3, 3),
            "index_add_1_thread_ms": round(t_add * 1e3, 3),
            "index_add_unused_thread_variant_ms": round(t_add_threads * 1e3, 3),
            "index_set_1_thread_ms": round(t_set * 1e3, 3),
            "uniform_8bit_quantize_ms": round(t_q * 1e3, 3),
        },
    }


def _per_launch(prof: dict, overhead_us: float) -> dict:
    """{kernel: (avg launch us net of the bracket overhead, algorithmic bytes per launch)}"""
    return {k: (max(v["total_ms"] / v["launches"] * 1e3 - overhead_us, 1e-3), v["algo_bytes"] / v["launches"]) for k, v in prof.items()}


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=30)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--streams", type=int, default=2,
                    help="HIP streams the buckets are spread over in the timed region (1 = strictly one after another)")
    ap.add_argument("--legs", default="buckets,t28,ring,chunks,outer,diloco,configs,staging",
                    help="comma list of t28 (carries value, roofline and the per-operation rows), buckets (configuration 2), ring, "
                         "chunks (ring chunks at their real sizes, one by one and segmented), outer, diloco, configs, staging")
    ap.add_argument("--t28-ops", default="",
                    help="comma list of substrings: the t28 leg runs only the operations whose name contains one of them "
                         "(uniform_8bit_quantize always runs: it carries the roofline)")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)", file=sys.stderr)
        return 2

    import torch
    from prime_amd import _lib, ops

    lib = _lib.load()          # raises if libprime_hip.so is not built: there is no fallback
    for opt in filter(None, os.environ.get("PRIME_HIP_OPTIONS", "").split(",")):   # tuning sweeps: name=value,...
        name, val = opt.split("=")
        _lib.set_option(name, int(val))
    legs = set(args.legs.split(","))
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    st = torch.cuda.current_stream(dev).cuda_stream
    ws = torch.empty(int(lib.prime_workspace_bytes()), dtype=torch.uint8, device=dev)
    _lib.check(lib.prime_workspace_init(ws.data_ptr(), ws.numel(), st), "workspace_init")

    def uniform(x, codes, lut, qp):
        _lib.check(lib.prime_uniform_8bit_quantize(x.data_ptr(), x.numel(), codes.data_ptr(), lut.data_ptr(), qp.data_ptr(),
                                                   ws.data_ptr(), st), "uniform_8bit_quantize")

    def ring_step(acc, codes_in, lut_in, codes_out, lut_out):
        _lib.check(lib.prime_ring_reduce_step(acc.data_ptr(), codes_in.data_ptr(), lut_in.data_ptr(), acc.numel(),
                                              codes_out.data_ptr(), lut_out.data_ptr(), None, ws.data_ptr(), st), "ring_step")

    # The device reaches its full clocks only after some milliseconds of continuous work (the first dozen
    # launches after an idle spell run up to a third slower): every timed region is preceded by about 20 ms
    # of untimed copies on the same stream, then by the warm-up steps, with no host synchronisation between.
    warm_src = torch.empty(1 << 26, dtype=torch.float32, device=dev).normal_()
    warm_dst = torch.empty_like(warm_src)

    def warm_device(n_copies=250):
        for _ in range(n_copies):
            lib.prime_copy_bytes(warm_dst.data_ptr(), warm_src.data_ptr(), warm_src.numel() * 4, st)

    def timed(step_fn, steps, warmup):
        warm_device()
        for _ in range(warmup):
            step_fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            step_fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / steps

    # A plain copy of known size (1 GiB read + 1 GiB written), untimed, and the FIRST launch of
    # copy_kernel in the process: the dispatch a profiler's FETCH_SIZE / WRITE_SIZE readings of the
    # other kernels are scaled against (prime_amd.rocprof_summary takes the first one).
    yard_src = torch.empty(1 << 28, dtype=torch.float32, device=dev).normal_()
    yard_dst = torch.empty_like(yard_src)
    _lib.check(lib.prime_copy_bytes(yard_dst.data_ptr(), yard_src.data_ptr(), yard_src.numel() * 4, st), "copy_bytes")
    torch.cuda.synchronize()
    del yard_src, yard_dst
    torch.cuda.empty_cache()

    # An event-bracketed launch cannot overlap its dispatch with the kernel before it, so a bracket can
    # read a few microseconds long.  Measured here, not assumed: twenty 256 MiB copies (long enough that
    # the host never falls behind, also under a profiler) bracketed, against the same twenty back to back.
    cal_src = torch.empty(1 << 26, dtype=torch.float32, device=dev).normal_()
    cal_dst = torch.empty_like(cal_src)

    def cal_copy():
        _lib.check(lib.prime_copy_bytes(cal_dst.data_ptr(), cal_src.data_ptr(), cal_src.numel() * 4, st), "copy_bytes")

    cal_wall = timed(cal_copy, 20, 3)
    _lib.profile_begin()
    for _ in range(20):
        cal_copy()
    cal_prof = _lib.profile_end()["copy_kernel"]
    overhead_from_copies_us = cal_prof["total_ms"] / cal_prof["launches"] * 1e3 - cal_wall * 1e6      # not clamped: a negative
    del cal_src, cal_dst                                                                             # reading must show
    event_overhead_us = max(0.0, overhead_from_copies_us)
    overhead_note = {"event_overhead_us_applied": round(event_overhead_us, 2),
                     "event_overhead_us_from_long_copies": round(overhead_from_copies_us, 2)}

    out = {
        "metric": "quantize+lookup & ring-reduce-step GB/s on 1 GPU; % of HBM peak; vs CPU ops",
        "value": None,
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": None,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {
            "workload": "uniform_8bit_quantize (statistics pass, then fused quantize + 256-bin lookup build) on one 2^28-element fp32 "
                        "tensor N(0, 1e-3) per step, three tensors and three code buffers (torch cuda generator, seeds 0..2) resident "
                        "in HBM and visited in rotation: 3 GiB pass through the 256 MB last-level cache between two visits of one tensor "
                        "(within a call the second pass finds the tensor's last 256 MiB in that cache, left there by the first: "
                        "8 of the 9 bytes per element come from or go to HBM)",
            "elements_per_step": N28,
            "algorithmic_bytes_per_element": 9,
            "n_bins": 256,
        },
    }
    bucket_kernel = None
    cpu_inputs = None

    if "buckets" in legs:
        # ---- config 2: 22 layer buckets, quantize + lookup per bucket ---------------------------
        buckets = [student_t3(BUCKET_ELEMS, dev, layer, 1e-4) for layer in range(N_LAYERS)]
        codes = [torch.empty(BUCKET_ELEMS, dtype=torch.uint8, device=dev) for _ in range(N_LAYERS)]
        luts = torch.empty((N_LAYERS, 256), dtype=torch.float32, device=dev)
        qps = torch.empty((N_LAYERS, 4), dtype=torch.float64, device=dev)

        def step_buckets():
            for i in range(N_LAYERS):
                uniform(buckets[i], codes[i], luts[i], qps[i])

        # The measured path: the buckets dealt over --streams HIP streams (prime_amd.ops.BucketPlan ->
        # prime_uniform_8bit_quantize_buckets), so one bucket's statistics pass overlaps its neighbours'
        # quantize pass and the launch ramps; results are those of the one-by-one loop.
        plan = ops.BucketPlan(buckets, codes, luts, qps, n_streams=args.streams)
        sec_pipelined = timed(plan.run, args.steps, args.warmup)
        elems = BUCKET_ELEMS * N_LAYERS
        value = 9.0 * elems / sec_pipelined / 1e9
        # The same buckets strictly one after another on one stream: the reference's order.
        sec = timed(step_buckets, args.steps, args.warmup)
        value_one_stream = 9.0 * elems / sec / 1e9
        # Third pass, one stream, with a start and a stop HIP event on every launch.
        _lib.profile_begin()
        for _ in range(args.steps):
            step_buckets()
        prof = _lib.profile_end()
        launches_per_bucket = sum(v["launches"] for v in prof.values()) / (args.steps * N_LAYERS)
        bracketed_us_per_bucket = sum(v["total_ms"] for v in prof.values()) * 1e3 / (args.steps * N_LAYERS)
        overhead_note["event_overhead_us_from_bucket_sequence"] = round(
            (bracketed_us_per_bucket - sec * 1e6 / N_LAYERS) / launches_per_bucket, 2)
        per = _per_launch(prof, event_overhead_us)
        # The same kernel with its input cold: the scales are known now, so quantize + lookup runs over
        # the 22 buckets in turn with nothing in between; each bucket was last touched 4.3 GB of traffic ago.
        scales = [float(ops.unpack_qparams(qps[i])["scale"]) for i in range(N_LAYERS)]

        def cold_pass():
            for i in range(N_LAYERS):
                _lib.check(lib.prime_quantize_lookup_u8(buckets[i].data_ptr(), BUCKET_ELEMS, scales[i], codes[i].data_ptr(),
                                                        luts[i].data_ptr(), ws.data_ptr(), st), "quantize_lookup")

        cold_pass()
        torch.cuda.synchronize()
        _lib.profile_begin()
        for _ in range(max(2, args.steps // 3)):
            cold_pass()
        cold = _per_launch(_lib.profile_end(), event_overhead_us)["quantize_kernel+hist"][0]
        dom_us, dom_bytes = per["quantize_kernel+hist"]
        bucket_kernel = {
            "workload": "one 51,380,224-element bucket (205 MB) of the step; the statistics pass has just streamed it, and "
                        "the 256 MB last-level cache serves part of this pass",
            "avg_launch_us": round(dom_us, 2), "achieved": round(dom_bytes / dom_us / 1e3, 1),
            "frac": round(dom_bytes / dom_us / 1e3 / HBM_PEAK_GBS, 4),
            "input_cold": {"what": "quantize + lookup with the scale given, over the 22 buckets in turn: every bucket comes from HBM",
                           "avg_launch_us": round(cold, 2), "achieved": round(dom_bytes / cold / 1e3, 1),
                           "frac": round(dom_bytes / cold / 1e3 / HBM_PEAK_GBS, 4)},
            "traffic": measured_traffic("cfg2_buckets_hbm_traffic.txt", "quantize_kernel<true, true, true, true"),
            "kernels": {k: {"avg_us": round(us, 2), "algo_GBps": round(b / us / 1e3, 1), "launches": prof[k]["launches"]}
                        for k, (us, b) in per.items()},
        }
        out["config_2_buckets"] = {
            "workload": "benchmark configuration 2: 22 per-layer pseudo-gradient buckets x 51,380,224 fp32 elements, Student-t(3)*1e-4 "
                        "(torch cuda generator, seed = layer), uniform_8bit_quantize bucket by bucket; cache-assisted: a 205 MB bucket "
                        "stays in the 256 MB last-level cache between its statistics pass and its quantize pass",
            "elements": elems, "algorithmic_bytes_per_element": 9,
            "one_stream": {"value": round(value_one_stream, 1), "unit": "GB/s", "ms": round(sec * 1e3, 4),
                           "frac_of_hbm_peak": round(value_one_stream / HBM_PEAK_GBS, 4)},
            "two_streams": {"value": round(value, 1), "unit": "GB/s", "ms": round(sec_pipelined * 1e3, 4), "streams": args.streams,
                            "frac_of_hbm_peak": round(value / HBM_PEAK_GBS, 4),
                            "what": "the buckets dealt over HIP streams: one bucket's statistics pass overlaps its neighbours' quantize pass"},
        }
        if "t28" not in legs:            # a profiler run of this leg alone: its figure stands in for the headline
            out.update({"value": round(value_one_stream, 1), "ms_per_step": round(sec * 1e3, 4)})
            out["config"]["workload"] = out["config_2_buckets"]["workload"]
        del buckets, codes, plan
        torch.cuda.empty_cache()

    if "t28" in legs:
        # ---- 2^28-element tensors: the size the target is quoted on; every operation of the path ----
        n28 = N28
        xs28 = []
        for seed in range(3):          # three tensors in rotation: 3 GiB between two visits of the same data
            g = torch.Generator(device=dev).manual_seed(seed)
            xs28.append(torch.randn(n28, device=dev, generator=g) * 1e-3)
        # outputs rotate too: a single reused 256 MiB code buffer would live in the last-level cache and its
        # writes would never reach HBM
        c28s = [torch.empty(n28, dtype=torch.uint8, device=dev) for _ in range(3)]
        o28s = [torch.empty(n28, device=dev) for _ in range(3)]
        cin28 = torch.empty(n28, dtype=torch.uint8, device=dev)
        l28 = torch.empty(256, dtype=torch.float32, device=dev)
        lin28 = torch.empty(256, dtype=torch.float32, device=dev)
        qp28 = torch.empty(4, dtype=torch.float64, device=dev)
        uniform(xs28[0], cin28, lin28, qp28)
        torch.cuda.synchronize()
        scale28 = float(ops.unpack_qparams(qp28)["scale"])
        import ctypes

        calls = {
            "stats (norm)": (4, lambda r: lib.prime_stats_f32(xs28[r % 3].data_ptr(), n28, qp28.data_ptr(), ws.data_ptr(), st)),
            "quantize_per_tensor_uint8 (a2)": (5, lambda r: lib.prime_quantize_u8(xs28[r % 3].data_ptr(), n28, ctypes.c_float(scale28), 128,
                                                                               c28s[r % 3].data_ptr(), st)),
            "average_buckets (a3)": (5, lambda r: lib.prime_average_buckets(xs28[r % 3].data_ptr(), cin28.data_ptr(), n28, 256, l28.data_ptr(),
                                                                            None, ws.data_ptr(), st)),
            "index_add (a4)": (9, lambda r: lib.prime_dequant_add(o28s[r % 3].data_ptr(), lin28.data_ptr(), cin28.data_ptr(), n28, st)),
            "index_set (a5)": (5, lambda r: lib.prime_dequant_set(o28s[r % 3].data_ptr(), lin28.data_ptr(), cin28.data_ptr(), n28, st)),
            "quantize + lookup, scale given (K2+K3)": (5, lambda r: lib.prime_quantize_lookup_u8(xs28[r % 3].data_ptr(), n28, ctypes.c_float(scale28),
                                                                                                c28s[r % 3].data_ptr(), l28.data_ptr(), ws.data_ptr(), st)),
            "uniform_8bit_quantize (a1)": (9, lambda r: lib.prime_uniform_8bit_quantize(xs28[r % 3].data_ptr(), n28, c28s[r % 3].data_ptr(), l28.data_ptr(),
                                                                                        qp28.data_ptr(), ws.data_ptr(), st)),
            "ring reduce step (a4 + a1)": (14, lambda r: lib.prime_ring_reduce_step(o28s[r % 3].data_ptr(), cin28.data_ptr(), lin28.data_ptr(), n28,
                                                                                   c28s[r % 3].data_ptr(), l28.data_ptr(), None, ws.data_ptr(), st)),
        }
        rows, uni_prof = {}, None
        only = [w for w in args.t28_ops.split(",") if w]
        for name, (bpe, fn) in calls.items():
            if only and name != "uniform_8bit_quantize (a1)" and not any(w in name for w in only):
                continue
            warm_device()
            for r in range(args.warmup):
                _lib.check(fn(r), name)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for r in range(args.steps):
                _lib.check(fn(r), name)
            torch.cuda.synchronize()
            wall = (time.perf_counter() - t0) / args.steps
            _lib.profile_begin()
            for r in range(args.steps):
                _lib.check(fn(r), name)
            prof28 = _lib.profile_end()
            per28 = _per_launch(prof28, event_overhead_us)
            kern_us = sum(us for us, _ in per28.values())
            rows[name] = {"bytes_per_element": bpe, "us": round(kern_us, 2), "GBps": round(bpe * n28 / kern_us / 1e3, 1),
                          "elements_per_s": round(n28 / (kern_us * 1e-6), 1), "frac_of_hbm_peak": round(bpe * n28 / kern_us / 1e3 / HBM_PEAK_GBS, 4),
                          "us_wall_back_to_back": round(wall * 1e6, 2),
                          "kernels": {k: {"avg_us": round(us, 2), "algo_GBps": round(b / us / 1e3, 1)} for k, (us, b) in per28.items()}}
            if name == "uniform_8bit_quantize (a1)":
                uni_prof = per28
        # What this device's memory delivers to the simplest kernels at the same size, for scale: reading
        # only (the statistics pass above), a plain copy, writing only (torch's fill).  HBM moves reads and
        # writes over one bus in turn, so a kernel that does both is bounded by the sum of the two times.
        def event_timed(fn):
            warm_device()
            for r in range(args.warmup):
                fn(r)
            evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(args.steps)]
            for r, (a, b) in enumerate(evs):
                a.record()
                fn(r)
                b.record()
            torch.cuda.synchronize()
            return sum(a.elapsed_time(b) for a, b in evs) / len(evs) * 1e3 - event_overhead_us
        copy_us = event_timed(lambda r: _lib.check(lib.prime_copy_bytes(o28s[r % 3].data_ptr(), xs28[r % 3].data_ptr(), n28 * 4, st), "copy"))
        fill_us = event_timed(lambda r: o28s[r % 3].fill_(1.0))
        yard = {"read_only_stats_kernel": {"GBps": rows["stats (norm)"]["GBps"], "frac_of_hbm_peak": rows["stats (norm)"]["frac_of_hbm_peak"]}
                if "stats (norm)" in rows else None,
                "copy_kernel_1GiB_to_1GiB": {"us": round(copy_us, 2), "GBps": round(8 * n28 / copy_us / 1e3, 1),
                                             "frac_of_hbm_peak": round(8 * n28 / copy_us / 1e3 / HBM_PEAK_GBS, 4)},
                "write_only_torch_fill_1GiB": {"us": round(fill_us, 2), "GBps": round(4 * n28 / fill_us / 1e3, 1),
                                               "frac_of_hbm_peak": round(4 * n28 / fill_us / 1e3 / HBM_PEAK_GBS, 4)}}
        dom_us, dom_bytes = uni_prof["quantize_kernel+hist"]
        cold_row = rows.get("quantize + lookup, scale given (K2+K3)")
        cold28 = None
        if cold_row:
            cold_us = cold_row["kernels"]["quantize_kernel+hist"]["avg_us"]
            cold28 = {"what": "prime_quantize_lookup_u8 (the same kernel, scale given, no statistics pass before it): every byte from HBM",
                      "avg_launch_us": cold_us, "achieved": round(dom_bytes / cold_us / 1e3, 1),
                      "frac": round(dom_bytes / cold_us / 1e3 / HBM_PEAK_GBS, 4)}
        uni, ring28 = rows["uniform_8bit_quantize (a1)"], rows.get("ring reduce step (a4 + a1)", {})
        # the headline: K calls of uniform_8bit_quantize back to back between two synchronisations
        step_s = uni["us_wall_back_to_back"] * 1e-6
        out.update({"value": round(9.0 * n28 / step_s / 1e9, 1), "ms_per_step": round(step_s * 1e3, 4),
                    "elements_per_s": round(n28 / step_s, 1), "frac_of_hbm_peak": round(9.0 * n28 / step_s / 1e9 / HBM_PEAK_GBS, 4),
                    # 8 of the 9 algorithmic bytes per element touch HBM: the quantize pass finds a quarter of the
                    # tensor in the last-level cache, where the statistics pass of the same call left it
                    "hbm_side": {"bytes_per_element": 8, "GBps": round(8.0 * n28 / step_s / 1e9, 1),
                                 "frac_of_hbm_peak": round(8.0 * n28 / step_s / 1e9 / HBM_PEAK_GBS, 4)}})
        if ring28:
            ring_s = ring28["us_wall_back_to_back"] * 1e-6
            out["ring_step_2p28"] = {
                "workload": "prime_ring_reduce_step on a 2^28-element accumulator (three in rotation) with a 2^28-code message: "
                            "acc += lut[codes] with the statistics of the result, then quantize + lookup; 14 bytes per element",
                "value": round(14.0 * n28 / ring_s / 1e9, 1), "unit": "GB/s", "ms_per_step": round(ring_s * 1e3, 4),
                "elements_per_s": round(n28 / ring_s, 1), "frac_of_hbm_peak": round(14.0 * n28 / ring_s / 1e9 / HBM_PEAK_GBS, 4),
                "sum_of_kernel_times": {"us": ring28["us"], "frac_of_hbm_peak": ring28["frac_of_hbm_peak"]}}
        out["tensor_2p28"] = {
            "workload": "2^28-element fp32 tensors N(0,1e-3), inputs and outputs three in rotation (3 GiB between two visits of the same "
                        "buffer); per operation: sum of its kernels' launch times (HIP events per launch), and wall time of "
                        "back-to-back calls",
            "value": uni["GBps"], "unit": "GB/s", "ms": round(uni["us"] / 1e3, 4), "elements_per_s": uni["elements_per_s"],
            "frac_of_hbm_peak": uni["frac_of_hbm_peak"],
            "ring_reduce_step": {"value": ring28["GBps"], "unit": "GB/s", "ms": round(ring28["us"] / 1e3, 4),
                                 "frac_of_hbm_peak": ring28["frac_of_hbm_peak"]} if ring28 else None,
            "operations": rows,
            "memory_yardsticks": yard,
        }
        out["roofline"] = {
            "bound": "hbm",
            "kernel": "quantize_kernel<aligned, nt loads, hist, walked from the end, non-temporal code stores, four-row tiles> "
                      "(quantize + 256-bin count / fixed-point sum histogram; 256 workgroups, the tiles of the tensor's cached end "
                      "visited spread among the others, the last 5 % of the tiles dealt on demand)",
            "workload": "inside uniform_8bit_quantize on 2^28-element tensors (1 GiB each; inputs and code buffers three in rotation: "
                        "nothing of either is left in the 256 MB last-level cache when the call starts).  Cache-assisted by the "
                        "call's own statistics pass, which reads the tensor's last 256 MiB without the non-temporal hint: this "
                        "pass takes that quarter of its reads from the last-level cache, interleaved with the three quarters from HBM; "
                        "input_cold is the same kernel with the scale given and nothing cached",
            "achieved": round(dom_bytes / dom_us / 1e3, 1),
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": round(dom_bytes / dom_us / 1e3 / HBM_PEAK_GBS, 4),
            "traffic": measured_traffic("uniform_2p28_hbm_traffic.txt", "quantize_kernel<true, true, true, true"),
            "algo_bytes_per_launch": 5 * n28,
            "avg_launch_us": round(dom_us, 2),
            **overhead_note,
            # what of it is HBM's own work: the 256 MiB the last-level cache serves taken off the bytes
            "hbm_side": {"bytes_per_launch": 5 * n28 - (256 << 20), "achieved": round((5 * n28 - (256 << 20)) / dom_us / 1e3, 1),
                         "frac": round((5 * n28 - (256 << 20)) / dom_us / 1e3 / HBM_PEAK_GBS, 4),
                         "note": "algorithmic bytes less the reads served by the last-level cache, over the same duration"},
            "input_cold": cold28,
            "on_the_buckets_of_the_step": bucket_kernel,
        }
        if not args.no_cpu_baseline:
            # what the CPU leg works on: the first tensor of the rotation, and for the ring hop the first quarter
            # (2^26 elements, configuration 3's chunk) of an accumulator with the message it received
            uniform(xs28[0], cin28, lin28, qp28)
            torch.cuda.synchronize()
            cpu_inputs = (xs28[0].cpu().numpy(), xs28[1][:RING_CHUNK].cpu().numpy().copy(), cin28[:RING_CHUNK].cpu().numpy().copy(),
                          lin28.cpu().numpy().copy())
        del xs28, c28s, cin28, o28s
        torch.cuda.empty_cache()
    elif bucket_kernel is not None:
        out["roofline"] = {"bound": "hbm", "kernel": "quantize_kernel+hist", "workload": bucket_kernel["workload"],
                           "achieved": bucket_kernel["achieved"], "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": bucket_kernel["frac"],
                           "traffic": measured_traffic("cfg2_buckets_hbm_traffic.txt", "quantize_kernel<true, true, true, true"), "algo_bytes_per_launch": 5 * BUCKET_ELEMS,
                           "avg_launch_us": bucket_kernel["avg_launch_us"], **overhead_note, "on_the_buckets_of_the_step": bucket_kernel}

    if "ring" in legs:
        # ---- config 3: ring reduce-scatter hops for W = 8 ranks' chunks ---------------------------
        chunks = []
        for r in range(RING_W):
            g = torch.Generator(device=dev).manual_seed(r)
            chunks.append(torch.randn(RING_CHUNK, device=dev, generator=g) * 1e-3)
        pristine = [c.clone() for c in chunks[1:]]
        cbuf = [torch.empty(RING_CHUNK, dtype=torch.uint8, device=dev) for _ in range(2)]
        lbuf = [torch.empty(256, dtype=torch.float32, device=dev) for _ in range(2)]
        qp = torch.empty(4, dtype=torch.float64, device=dev)

        def hops():
            for r in range(1, RING_W):
                ring_step(chunks[r], cbuf[(r - 1) % 2], lbuf[(r - 1) % 2], cbuf[r % 2], lbuf[r % 2])

        def restore():
            for c, p in zip(chunks[1:], pristine):
                c.copy_(p)

        uniform(chunks[0], cbuf[0], lbuf[0], qp)
        ring_steps = max(2, args.steps // 2)
        hop_sec = []
        for it in range(args.warmup + ring_steps):
            restore()                   # every pass starts from the ranks' own data
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            hops()
            torch.cuda.synchronize()
            if it >= args.warmup:
                hop_sec.append((time.perf_counter() - t0) / (RING_W - 1))
        hop = statistics.mean(hop_sec)
        restore()
        _lib.profile_begin()
        hops()
        rprof = _lib.profile_end()
        ring_gbs = 14.0 * RING_CHUNK / hop / 1e9
        out["ring_step"] = {
            "workload": "benchmark configuration 3: W=8 ranks, 2^26-element chunks N(0,1e-3) (seed = rank); per hop: "
                        "acc += lut[codes]; uniform_8bit_quantize(acc)",
            "value": round(ring_gbs, 1),
            "unit": "GB/s",
            "algorithmic_bytes_per_element": 14,
            "ms_per_hop": round(hop * 1e3, 4),
            "elements_per_s": round(RING_CHUNK / hop, 1),
            "frac_of_hbm_peak": round(ring_gbs / HBM_PEAK_GBS, 4),
            "kernels": kernel_table(rprof, event_overhead_us),
        }
        del chunks, pristine, cbuf
        torch.cuda.empty_cache()

    if "chunks" in legs:
        # ---- the sizes the ring really runs at: a layer bucket is cut into 2 W chunks (collectives.cpp:89-90) -----
        # one ring hop / one uniform_8bit_quantize per chunk, chunk after chunk (three launches each), against all
        # W = 8 ranks' chunks of one step of the lock-stepped ring in ONE segmented call (three launches in all).
        # Three sets of tensors in rotation, so that a set is not simply served by the last-level cache.
        def chunk_rows(label, sizes, rot):
            res = {}
            tot = sum(sizes)
            g = torch.Generator(device=dev).manual_seed(len(sizes) * 1000 + sizes[0] % 997)
            for kind, bpe in ((ops.SEG_UNIFORM, 9), (ops.SEG_REDUCE, 14)):
                plans, singles = [], []
                for _ in range(rot):
                    xs = [torch.randn(n, device=dev, generator=g) * 1e-3 for n in sizes]
                    cs = [torch.empty(n, dtype=torch.uint8, device=dev) for n in sizes]
                    ls = torch.empty((len(sizes), 256), device=dev)
                    if kind == ops.SEG_UNIFORM:
                        plans.append(ops.SegmentPlan(kind, xs, codes=cs, luts=ls))

                        def one(xs=xs, cs=cs, ls=ls):
                            for x, c, l in zip(xs, cs, ls):
                                _lib.check(lib.prime_uniform_8bit_quantize(x.data_ptr(), x.numel(), c.data_ptr(), l.data_ptr(), None,
                                                                           ws.data_ptr(), st), "uniform")
                    else:
                        cin, lin = ops.uniform_8bit_quantize_segmented([torch.randn(n, device=dev, generator=g) * 1e-3 for n in sizes])
                        plans.append(ops.SegmentPlan(kind, xs, cin, list(lin), codes=cs, luts=ls))

                        def one(xs=xs, cin=cin, lin=lin, cs=cs, ls=ls):
                            for a, ci, li, c, l in zip(xs, cin, lin, cs, ls):
                                ring_step(a, ci, li, c, l)
                    singles.append(one)
                k = [0]

                def run_seg():
                    plans[k[0] % rot].run()
                    k[0] += 1

                def run_one():
                    singles[k[0] % rot]()
                    k[0] += 1

                t_seg = timed(run_seg, args.steps * 2, args.warmup)
                t_one = timed(run_one, args.steps * 2, args.warmup)
                _lib.profile_begin()
                for _ in range(max(3, args.steps // 2)):
                    run_seg()
                kern = kernel_table(_lib.profile_end(), event_overhead_us)
                res["uniform_8bit_quantize" if kind == ops.SEG_UNIFORM else "ring_reduce_step"] = {
                    "bytes_per_element": bpe,
                    "segmented": {"us": round(t_seg * 1e6, 2), "GBps": round(bpe * tot / t_seg / 1e9, 1),
                                  "frac_of_hbm_peak": round(bpe * tot / t_seg / 1e9 / HBM_PEAK_GBS, 4), "kernels": kern},
                    "one_by_one": {"us": round(t_one * 1e6, 2), "GBps": round(bpe * tot / t_one / 1e9, 1),
                                   "frac_of_hbm_peak": round(bpe * tot / t_one / 1e9 / HBM_PEAK_GBS, 4),
                                   "us_per_tensor": round(t_one * 1e6 / len(sizes), 2)},
                    "speedup": round(t_one / t_seg, 2)}
                del plans, singles
                torch.cuda.empty_cache()
            return {"tensors": len(sizes), "elements_each": sizes[0], "elements": tot, **res}

        out["ring_chunks"] = {
            "workload": "N(0, 1e-3) chunks, three sets in rotation; one_by_one: the one-tensor entry point per chunk (three launches each); "
                        "segmented: all chunks in one call (three launches in all), results bit-identical",
            "config_2_bucket_over_16 x W=8": chunk_rows("cfg2", [RING_CHUNK_CFG2] * RING_W, 3),
            "config_4_bucket_over_16 x W=8": chunk_rows("cfg4", [RING_CHUNK_CFG4] * RING_W, 3),
            "64 x 2^20": chunk_rows("2p20", [1 << 20] * 64, 2),
        }

    if "outer" in legs:
        # ---- the callers either side of the path: pseudo-gradient and outer optimizer step -----------
        n_o = 1 << 28
        g = torch.Generator(device=dev).manual_seed(7)
        outer_p = torch.randn(n_o, device=dev, generator=g)
        inner_p = outer_p + torch.randn(n_o, device=dev, generator=g) * 1e-3
        grad = torch.empty(n_o, device=dev)
        mom = torch.zeros(n_o, device=dev)
        c_o = torch.empty(n_o, dtype=torch.uint8, device=dev)
        l_o = torch.empty(256, dtype=torch.float32, device=dev)
        q_o = torch.empty(4, dtype=torch.float64, device=dev)

        def pg():
            _lib.check(lib.prime_pseudo_gradient_f32(outer_p.data_ptr(), inner_p.data_ptr(), n_o, 8.0, grad.data_ptr(), st), "pg")

        def sgd():
            _lib.check(lib.prime_outer_sgd_nesterov_f32(outer_p.data_ptr(), mom.data_ptr(), grad.data_ptr(), inner_p.data_ptr(),
                                                        n_o, 0.7, 0.9, 0, st), "sgd")

        def sgd_codes():
            _lib.check(lib.prime_outer_sgd_nesterov_u8(outer_p.data_ptr(), mom.data_ptr(), c_o.data_ptr(), l_o.data_ptr(),
                                                       inner_p.data_ptr(), n_o, 0.7, 0.9, 0, st), "sgd_codes")

        t_pg = timed(pg, args.steps, args.warmup)
        uniform(grad, c_o, l_o, q_o)
        t_sgd = timed(sgd, args.steps, args.warmup)
        t_sgdc = timed(sgd_codes, args.steps, args.warmup)
        out["outer_step"] = {
            "workload": "2^28 fp32 parameters: pseudo-gradient (outer - inner) / W; SGD-Nesterov outer step fused with the "
                        "copy to the inner model, from an fp32 gradient and from uint8 codes + lookup",
            "pseudo_gradient": {"GBps": round(12.0 * n_o / t_pg / 1e9, 1), "bytes_per_element": 12, "ms": round(t_pg * 1e3, 4),
                                "frac_of_hbm_peak": round(12.0 * n_o / t_pg / 1e9 / HBM_PEAK_GBS, 4)},
            "outer_sgd_nesterov": {"GBps": round(24.0 * n_o / t_sgd / 1e9, 1), "bytes_per_element": 24, "ms": round(t_sgd * 1e3, 4),
                                   "frac_of_hbm_peak": round(24.0 * n_o / t_sgd / 1e9 / HBM_PEAK_GBS, 4)},
            "outer_sgd_nesterov_from_codes": {"GBps": round(21.0 * n_o / t_sgdc / 1e9, 1), "bytes_per_element": 21,
                                              "ms": round(t_sgdc * 1e3, 4),
                                              "frac_of_hbm_peak": round(21.0 * n_o / t_sgdc / 1e9 / HBM_PEAK_GBS, 4)},
        }
        # a chunk's first visit in the ring with the pseudo-gradient formed on the way (config 3's chunk
        # shape), against pseudo-gradient, then ring step as separate calls
        n_c = RING_CHUNK
        ci = torch.empty(n_c, dtype=torch.uint8, device=dev)
        li = torch.empty(256, dtype=torch.float32, device=dev)
        uniform(grad[:n_c], ci, li, q_o)
        co = torch.empty(n_c, dtype=torch.uint8, device=dev)
        lo = torch.empty(256, dtype=torch.float32, device=dev)
        # eight chunk-sized windows, so that no pass finds its operands in the last-level cache
        wins = [slice(k * n_c, (k + 1) * n_c) for k in range(n_o // n_c)]

        def touch(with_msg):
            for w in wins:
                _lib.check(lib.prime_ring_first_touch(outer_p[w].data_ptr(), inner_p[w].data_ptr(), n_c, 8.0,
                                                      ci.data_ptr() if with_msg else None, li.data_ptr() if with_msg else None,
                                                      1.0, grad[w].data_ptr(), co.data_ptr(), lo.data_ptr(), None, ws.data_ptr(), st),
                           "first touch")

        def separate(with_msg):
            for w in wins:
                _lib.check(lib.prime_pseudo_gradient_f32(outer_p[w].data_ptr(), inner_p[w].data_ptr(), n_c, 8.0,
                                                         grad[w].data_ptr(), st), "pg")
                if with_msg:
                    ring_step(grad[w], ci, li, co, lo)
                else:
                    uniform(grad[w], co, lo, q_o)

        ft = {}
        # (without a message prime_ring_first_touch itself takes the separate kernels: they are the faster route)
        for name, with_msg, fused_b, sep_b in (("send_first", False, 21, 21), ("with_message", True, 18, 26)):
            t_f = timed(lambda: touch(with_msg), args.steps, args.warmup) / len(wins)
            t_s = timed(lambda: separate(with_msg), args.steps, args.warmup) / len(wins)
            ft[name] = {"fused_ms": round(t_f * 1e3, 4), "fused_bytes_per_element": fused_b,
                        "fused_GBps": round(fused_b * n_c / t_f / 1e9, 1),
                        "fused_frac_of_hbm_peak": round(fused_b * n_c / t_f / 1e9 / HBM_PEAK_GBS, 4),
                        "separate_ms": round(t_s * 1e3, 4), "separate_bytes_per_element": sep_b,
                        "speedup": round(t_s / t_f, 3)}
        out["outer_step"]["ring_first_touch"] = dict(
            workload="2^26-element chunks: grad = (outer - inner) / W [+ lut[codes]] and uniform_8bit_quantize(grad) in two "
                     "passes, against prime_pseudo_gradient_f32 followed by prime_uniform_8bit_quantize / prime_ring_reduce_step",
            **ft)
        del outer_p, inner_p, grad, mom, c_o, ci, co
        torch.cuda.empty_cache()

    if "diloco" in legs:
        # ---- a whole outer step of W simulated workers: pseudo-gradient, ring all-reduce, outer step --
        from prime_amd import ring

        W_d, n_d = 4, 8 * RING_CHUNK                   # 2 W chunks of config 3's chunk size per worker
        g = torch.Generator(device=dev).manual_seed(11)
        outers, inners, grads, moms = [], [], [], []
        for r in range(W_d):
            o = torch.randn(n_d, device=dev, generator=g)
            outers.append(o)
            inners.append(o + torch.randn(n_d, device=dev, generator=g) * 1e-3)
            grads.append(torch.empty(n_d, device=dev))
            moms.append(torch.zeros(n_d, device=dev))
        csz = n_d // (2 * W_d)

        def step_plain():
            for r in range(W_d):
                ops.pseudo_gradient_(grads[r], outers[r], inners[r], float(W_d))
            ring.ring_allreduce_simulated(grads)
            for r in range(W_d):
                ops.outer_sgd_nesterov_(outers[r], moms[r], grads[r], inners[r], 0.7, 0.9, False)

        def step_fused():
            final = ring.ring_allreduce_simulated(grads, sources=list(zip(outers, inners)), world_size=float(W_d), keep_codes=True)
            for r in range(W_d):
                for c, (cd, lt) in enumerate(final[r]):
                    sl = slice(c * csz, (c + 1) * csz)
                    ops.outer_sgd_nesterov_codes_(outers[r][sl], moms[r][sl], cd, lt, inners[r][sl], 0.7, 0.9, False)

        d_steps = max(2, args.steps // 3)
        t_plain = timed(step_plain, d_steps, 1)
        t_fused = timed(step_fused, d_steps, 1)
        nb_d = 2 * W_d
        plain_b = (12 * nb_d + 2 * 9 + (nb_d - 2) * 14 + (nb_d - 2) * 10 + 2 * 5 + 24 * nb_d) / nb_d
        fused_b = (2 * 21 + (nb_d - 2) * 18 + (nb_d - 2) * 3 + 21 * nb_d) / nb_d
        out["diloco_outer_step"] = {
            "workload": f"W={W_d} simulated workers of {n_d} fp32 parameters each ({nb_d} chunks of 2^26): pseudo-gradient, "
                        "uint8 ring all-reduce (both phases), SGD-Nesterov outer step and copy to the inner model",
            "separate_kernels": {"ms": round(t_plain * 1e3, 3), "bytes_per_element_per_worker": round(plain_b, 2),
                                 "GBps": round(plain_b * n_d * W_d / t_plain / 1e9, 1)},
            "fused": {"ms": round(t_fused * 1e3, 3), "bytes_per_element_per_worker": round(fused_b, 2),
                      "GBps": round(fused_b * n_d * W_d / t_fused / 1e9, 1),
                      "what": "pseudo-gradient formed at a chunk's first visit, all-gather in the code domain, outer step from codes"},
            "speedup": round(t_plain / t_fused, 3),
            "parameters_per_s_fused": round(n_d * W_d / t_fused, 1),
        }
        del outers, inners, grads, moms
        torch.cuda.empty_cache()

    if "configs" in legs:
        # ---- the other benchmark configurations, one figure each ---------------------------------------
        import numpy as np

        cfgs = {}

        def dequant(o, lut_t, codes_t):
            _lib.check(lib.prime_dequant_set(o.data_ptr(), lut_t.data_ptr(), codes_t.data_ptr(), o.numel(), st), "dequant_set")

        # config 1: 2^24 elements N(0, 1e-3), quantize -> dequantize round trip (14 B/element; 64 MiB:
        # the tensor stays in the 256 MB last-level cache between the passes)
        n1 = 1 << 24
        g = torch.Generator(device=dev).manual_seed(0)
        x1 = torch.randn(n1, device=dev, generator=g) * 1e-3
        c1 = torch.empty(n1, dtype=torch.uint8, device=dev)
        o1 = torch.empty(n1, device=dev)
        l1 = torch.empty(256, device=dev)
        q1 = torch.empty(4, dtype=torch.float64, device=dev)

        def cfg1():
            uniform(x1, c1, l1, q1)
            dequant(o1, l1, c1)

        t1 = timed(cfg1, args.steps * 5, args.warmup)
        cfgs["config_1_round_trip_2p24"] = {"us": round(t1 * 1e6, 2), "bytes_per_element": 14, "GBps": round(14.0 * n1 / t1 / 1e9, 1),
                                           "frac_of_hbm_peak": round(14.0 * n1 / t1 / 1e9 / HBM_PEAK_GBS, 4),
                                           "note": "cache-assisted: 64 MiB fits the last-level cache"}
        del x1, c1, o1

        # config 4: 1.25e9 elements in 42 buckets (29,761,904 each, the last 32 longer), N(0, 5e-4) with
        # 0.01 % of entries at +-50 sigma; quantize + lookup over --streams streams, then dequantize
        sizes4 = [29_761_904] * 41 + [29_761_904 + 32]
        xs4 = []
        for b, nb4 in enumerate(sizes4):
            g = torch.Generator(device=dev).manual_seed(400 + b)
            x = torch.randn(nb4, device=dev, generator=g) * 5e-4
            pos = torch.randint(0, nb4, (nb4 // 10000,), device=dev, generator=g)
            sign = torch.randint(0, 2, (nb4 // 10000,), device=dev, generator=g).float() * 2 - 1
            x[pos] = sign * (50 * 5e-4)
            xs4.append(x)
        cs4 = [torch.empty(nb4, dtype=torch.uint8, device=dev) for nb4 in sizes4]
        os4 = [torch.empty(nb4, device=dev) for nb4 in sizes4]
        l4 = torch.empty((42, 256), device=dev)
        q4 = torch.empty((42, 4), dtype=torch.float64, device=dev)
        plan4 = ops.BucketPlan(xs4, cs4, l4, q4, n_streams=args.streams)

        def cfg4():
            plan4.run()
            for b in range(42):
                dequant(os4[b], l4[b], cs4[b])

        steps4 = max(2, args.steps // 3)
        t4 = timed(cfg4, steps4, 1)
        cfgs["config_4_shard_42_buckets"] = {"ms": round(t4 * 1e3, 3), "bytes_per_element": 14, "elements": sum(sizes4),
                                            "GBps": round(14.0 * sum(sizes4) / t4 / 1e9, 1),
                                            "frac_of_hbm_peak": round(14.0 * sum(sizes4) / t4 / 1e9 / HBM_PEAK_GBS, 4)}
        del xs4, cs4, os4, plan4
        torch.cuda.empty_cache()

        # config 5: 2,000 small tensors N(1, 1e-2), sizes U[1, 65536], in one launch; the edge tensors
        rng = np.random.default_rng(5)
        sizes5 = rng.integers(1, 65536, 2000, endpoint=True)
        off5 = torch.from_numpy(np.concatenate([[0], np.cumsum(sizes5)]).astype(np.int64)).to(dev)
        tot5 = int(sizes5.sum())
        g = torch.Generator(device=dev).manual_seed(5)
        x5 = torch.randn(tot5, device=dev, generator=g) * 1e-2 + 1
        c5 = torch.empty(tot5, dtype=torch.uint8, device=dev)
        l5 = torch.empty((2000, 256), device=dev)
        q5 = torch.empty((2000, 4), dtype=torch.float64, device=dev)

        def cfg5():
            _lib.check(lib.prime_uniform_8bit_quantize_batched(x5.data_ptr(), off5.data_ptr(), 2000, c5.data_ptr(), l5.data_ptr(),
                                                               q5.data_ptr(), st), "batched")

        t5 = timed(cfg5, args.steps * 3, args.warmup)
        edge = {}
        n20 = 1 << 20
        g = torch.Generator(device=dev).manual_seed(50)
        half = torch.randn(n20, device=dev, generator=g) * 1e-3
        half[torch.rand(n20, device=dev, generator=g) < 0.5] = 0
        tail = torch.randn((1 << 24) + 7, device=dev, generator=g) * 1e-3
        for name, x in (("constant_2p20", torch.full((n20,), 0.25, device=dev)), ("zeros_2p20", torch.zeros(n20, device=dev)),
                        ("half_zeros_2p20", half), ("tail_2p24_plus_7", tail)):
            ce = torch.empty(x.numel(), dtype=torch.uint8, device=dev)
            te = timed(lambda: uniform(x, ce, l1, q1), args.steps * 5, args.warmup)
            edge[name] = {"us": round(te * 1e6, 2), "GBps": round(9.0 * x.numel() / te / 1e9, 1)}
        cfgs["config_5_small_and_edge_tensors"] = {
            "batched_2000_tensors": {"us": round(t5 * 1e6, 2), "elements": tot5, "bytes_per_element": 9,
                                     "GBps": round(9.0 * tot5 / t5 / 1e9, 1),
                                     "frac_of_hbm_peak": round(9.0 * tot5 / t5 / 1e9 / HBM_PEAK_GBS, 4)},
            "edge": edge, "note": "the 2^20-element tensors (4 MiB) run from cache and are bound by launch latency"}
        out["other_configs"] = cfgs

    if "staging" in legs:
        # ---- the PCIe side of a host transport: codes + lookup through pinned host double buffers ---------
        from prime_amd import wire

        def staging_at(n_s):
            stage = wire.HostStage(dev, n_s)
            g = torch.Generator(device=dev).manual_seed(21)
            accs = [torch.randn(n_s, device=dev, generator=g) * 1e-3 for _ in range(4)]
            c_s, l_s = ops.uniform_8bit_quantize(accs[0])
            hops_s = 6

            def d2h_only():
                for k in range(hops_s):
                    stage.post_send(k, c_s, l_s)
                    stage.take_send(k)

            def h2d_only():
                for k in range(hops_s):
                    stage.recv_buffers(k)
                    stage.to_device(k)
                    stage.release(k)

            def kernels_only():
                cc, ll = c_s, l_s
                for k in range(hops_s):
                    cc, ll = ops.ring_reduce_step(accs[k % 4], cc, ll)

            def staged_hops():
                # hop k: received message (host) -> device, ring step, result -> host; the transport hands the
                # sender's slot straight to the receiver (no copy), so what is timed is PCIe and kernels
                cc, ll = c_s, l_s
                stage.post_send(0, cc, ll)
                for k in range(hops_s):
                    lut_h, codes_h = stage.take_send(k)
                    rl, rc = stage.recv_buffers(k)
                    rl.copy_(lut_h)
                    stage.recv_codes[k % stage.depth], stage.send_codes[k % stage.depth] = codes_h, rc     # swap the slots
                    dc, dl = stage.to_device(k)
                    cc, ll = ops.ring_reduce_step(accs[k % 4], dc, dl)
                    stage.release(k)
                    stage.post_send(k + 1, cc, ll)
                stage.take_send(hops_s)

            reps_s = 3 if n_s >= (1 << 24) else 10
            t_d2h = timed(d2h_only, reps_s, 1) / hops_s
            t_h2d = timed(h2d_only, reps_s, 1) / hops_s
            t_k = timed(kernels_only, reps_s, 1) / hops_s
            t_st = timed(staged_hops, reps_s, 1) / hops_s
            msg_bytes = n_s + 1024
            return {
                "message_bytes": msg_bytes, "fp32_chunk_bytes": 4 * n_s,
                "device_to_host": {"ms": round(t_d2h * 1e3, 3), "GBps": round(msg_bytes / t_d2h / 1e9, 1)},
                "host_to_device": {"ms": round(t_h2d * 1e3, 3), "GBps": round(msg_bytes / t_h2d / 1e9, 1)},
                "ring_step_kernels_ms": round(t_k * 1e3, 3),
                "staged_hop_ms": round(t_st * 1e3, 3),
            }

        out["host_staging"] = {
            "workload": "ring hops on 2^26-element chunks with every message through pinned host buffers "
                        "(device -> host, host -> device on a copy stream); the host-to-host transport itself is not timed",
            **staging_at(RING_CHUNK),
            "note": "a hop is bound by the two PCIe copies of the uint8 codes; staging fp32 would move four times as much",
            "chunk_of_a_config_2_bucket_at_W8": {"elements": BUCKET_ELEMS // 16, **staging_at(BUCKET_ELEMS // 16)},
        }

    if not args.no_cpu_baseline:
        if cpu_inputs is None:           # the t28 leg did not run: one configuration-2 bucket, drawn as the GPU leg draws it
            b0 = student_t3(BUCKET_ELEMS, dev, 0, 1e-4)
            c0, l0 = ops.uniform_8bit_quantize(b0[:RING_CHUNK // 4])
            cpu_inputs = (b0.cpu().numpy(), b0[RING_CHUNK // 4: RING_CHUNK // 2].cpu().numpy().copy(), c0.cpu().numpy(), l0.cpu().numpy())
            what = "one 51,380,224-element Student-t(3)*1e-4 bucket of configuration 2"
            del b0
        else:
            what = "the first 2^28-element N(0, 1e-3) tensor of the GPU leg's rotation"
        out["cpu_baseline"] = cpu_baseline(*cpu_inputs, what=what, reps=3)
        out["gpu_over_cpu"] = round(out["value"] / out["cpu_baseline"]["value"], 1) if out["value"] and out["cpu_baseline"]["value"] else None

    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
