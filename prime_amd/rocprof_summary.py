"""Short text summaries of rocprofv3 CSV output for the kernels of libprime_hip.so.

    python -m prime_amd.rocprof_summary trace    <dir> [--title T] [--command C]
    python -m prime_amd.rocprof_summary traffic  <fetch_dir> <write_dir> [--title T] [--command C]
    python -m prime_amd.rocprof_summary counters <dir> [<dir> ...] [--title T] [--command C]
    (all three: [--bench-json FILE] appends the figures bench.py printed in that run, [--note TEXT])

<dir> is what ``rocprofv3 ... --output-format csv -d <dir> -o bench`` wrote (it may put the files
one level down, in a directory named after the host).  ``trace`` reads bench_kernel_trace.csv of a
``--kernel-trace`` run, the other two read bench_counter_collection.csv of ``--pmc`` runs.

Kernel rows are grouped by (kernel name with template arguments, grid size); torch's own
kernels (input generation) are left out.

``traffic``: FETCH_SIZE and WRITE_SIZE are KiB per dispatch as the L2 reports them.  They are
scaled by what the same counters read for a copy of known size: the FIRST dispatch of copy_kernel
in the run, which bench.py makes a 1 GiB copy (1,048,576 KiB read and as much written) before
anything else.  scaled bytes = FETCH * (1048576 / FETCH_copy) + WRITE * (1048576 / WRITE_copy), in KiB.
"""
from __future__ import annotations

import argparse
import collections
import csv
import re
import sys
from pathlib import Path

YARDSTICK_KIB = 1048576.0


def _find(directory: str, name: str) -> Path:
    hits = sorted(Path(directory).rglob(name))
    if not hits:
        raise SystemExit(f"{name} not found under {directory}")
    return hits[0]


def short(name: str) -> str:
    name = name.replace("(anonymous namespace)::", "")
    name = re.sub(r"^void ", "", name)
    m = re.match(r"([A-Za-z_0-9:]+(<[^(]*>)?)\(", name)
    return (m.group(1) if m else name)[:96]


def _ours(name: str) -> bool:
    return "at::native" not in name and "rocclr" not in name and "elementwise_kernel" not in name and "hipcub" not in name \
        and "rocprim" not in name


def trace(directory: str) -> str:
    rows = [r for r in csv.DictReader(open(_find(directory, "bench_kernel_trace.csv"))) if _ours(r["Kernel_Name"])]
    acc = collections.defaultdict(list)
    for r in rows:
        grid = int(r["Grid_Size_X"]) // max(int(r["Workgroup_Size_X"]), 1)
        acc[(short(r["Kernel_Name"]), grid)].append((int(r["End_Timestamp"]) - int(r["Start_Timestamp"])) / 1e3)
    lines = [f"{'kernel':96s} {'wgs':>5s} {'calls':>6s} {'avg_us':>9s} {'median':>9s} {'min_us':>9s} {'max_us':>9s} {'total_ms':>9s}"]
    for (name, grid), d in sorted(acc.items(), key=lambda kv: -sum(kv[1])):
        d = sorted(d)
        lines.append(f"{name:96s} {grid:5d} {len(d):6d} {sum(d) / len(d):9.2f} {d[len(d) // 2]:9.2f} {d[0]:9.2f} {d[-1]:9.2f} {sum(d) / 1e3:9.3f}")
    return "\n".join(lines)


def _counter_rows(directory: str):
    return [r for r in csv.DictReader(open(_find(directory, "bench_counter_collection.csv"))) if _ours(r["Kernel_Name"])]


def _per_kernel(rows, counter: str):
    """{(kernel, workgroups): [value per dispatch]} for one counter; a dispatch's value is the sum
    over the rows it has for that counter (one per shader engine or XCD on some versions)."""
    per_dispatch = collections.defaultdict(float)
    meta = {}
    for r in rows:
        if r["Counter_Name"] != counter:
            continue
        d = int(r["Dispatch_Id"])
        per_dispatch[d] += float(r["Counter_Value"])
        meta[d] = (short(r["Kernel_Name"]), int(r["Grid_Size"]) // max(int(r["Workgroup_Size"]), 1))
    acc = collections.defaultdict(list)
    for d in sorted(per_dispatch):
        acc[meta[d]].append((d, per_dispatch[d]))
    return acc


def traffic(fetch_dir: str, write_dir: str) -> str:
    fe = _per_kernel(_counter_rows(fetch_dir), "FETCH_SIZE")
    wr = _per_kernel(_counter_rows(write_dir), "WRITE_SIZE")

    def yardstick(acc, what):
        copies = [v for (name, _), vals in acc.items() if name.startswith("copy_kernel") for v in vals]
        if not copies:
            raise SystemExit(f"no copy_kernel dispatch in the {what} run: nothing to scale against")
        return min(copies)[1]            # lowest dispatch id = the first copy = the 1 GiB yardstick

    cf, cw = yardstick(fe, "FETCH_SIZE"), yardstick(wr, "WRITE_SIZE")
    ff, fw = YARDSTICK_KIB / cf, YARDSTICK_KIB / cw
    lines = [f"yardstick (first copy_kernel dispatch, 1 GiB each way): FETCH_SIZE reads {cf:.1f} KiB -> factor {ff:.4f}; "
             f"WRITE_SIZE reads {cw:.1f} KiB -> factor {fw:.4f}",
             "per dispatch, averaged over the dispatches of that (kernel, workgroups) group in the run:", "",
             f"{'kernel':96s} {'wgs':>5s} {'n':>4s} {'FETCH_KiB':>12s} {'WRITE_KiB':>12s} {'read_MB':>10s} {'written_MB':>10s} {'total_MB':>10s}"]
    for key in sorted(set(fe) | set(wr), key=lambda k: (k[0], k[1])):
        if key[0].startswith("fill_zero"):
            continue
        f = [v for _, v in fe.get(key, [])]
        w = [v for _, v in wr.get(key, [])]
        fa = sum(f) / len(f) if f else 0.0
        wa = sum(w) / len(w) if w else 0.0
        rmb, wmb = fa * ff * 1024 / 1e6, wa * fw * 1024 / 1e6
        lines.append(f"{key[0]:96s} {key[1]:5d} {max(len(f), len(w)):4d} {fa:12.1f} {wa:12.1f} {rmb:10.2f} {wmb:10.2f} {rmb + wmb:10.2f}")
    return "\n".join(lines)


def counters(directories) -> str:
    rows = [r for d in directories for r in _counter_rows(d)]
    names = sorted({r["Counter_Name"] for r in rows})
    table = {c: _per_kernel(rows, c) for c in names}
    keys = sorted({k for c in names for k in table[c]}, key=lambda k: (k[0], k[1]))
    lines = ["per dispatch, averaged over the dispatches of that (kernel, workgroups) group:", ""]
    for key in keys:
        if key[0].startswith("fill_zero"):
            continue
        lines.append(f"{key[0]}  [{key[1]} workgroups]")
        for c in names:
            vals = [v for _, v in table[c].get(key, [])]
            if vals:
                lines.append(f"    {c:28s} {sum(vals) / len(vals):18.1f}   (n={len(vals)})")
    return "\n".join(lines)


def bench_excerpt(path: str) -> str:
    """What bench.py itself printed in the profiled run (its single JSON line): the figures it took
    from HIP events, to set beside the profiler's."""
    import json

    text = [ln for ln in open(path).read().splitlines() if ln.startswith("{")]
    if not text:
        return "(no JSON line in " + path + ")"
    d = json.loads(text[-1])
    out = ["", "bench.py's own figures from the same run (HIP events around each launch):"]
    if d.get("value") is not None:
        out.append(f"  value={d['value']} GB/s ms_per_step={d['ms_per_step']} frac_of_hbm_peak={d.get('frac_of_hbm_peak')}")
    r = d.get("roofline")
    if r:
        out.append("  roofline: " + json.dumps({k: v for k, v in r.items() if k not in ("on_the_buckets_of_the_step", "workload", "kernel")}))
        b = r.get("on_the_buckets_of_the_step")
        if b:
            out.append("  bucket kernel: " + json.dumps({k: v for k, v in b.items() if k not in ("workload", "kernels")}))
            for k, v in b["kernels"].items():
                out.append(f"    {k:30s} avg_us={v['avg_us']:9.2f} algo_GBps={v['algo_GBps']}")
    t = d.get("tensor_2p28")
    if t:
        for name, v in t["operations"].items():
            out.append(f"  2^28 {name:42s} us={v['us']:9.2f} GBps={v['GBps']:8.1f} frac={v['frac_of_hbm_peak']:.4f}  " +
                       " ".join(f"{k}={kv['avg_us']}" for k, kv in v["kernels"].items()))
    for key in ("ring_step",):
        if key in d:
            out.append(f"  {key}: value={d[key]['value']} GB/s frac_of_hbm_peak={d[key]['frac_of_hbm_peak']} ms_per_hop={d[key]['ms_per_hop']}")
            for k, v in d[key]["kernels"].items():
                out.append(f"    {k:30s} avg_us={v['avg_us']:9.2f} algo_GBps={v['algo_GBps']}")
    if "other_configs" in d:
        out.append("  other_configs: " + json.dumps(d["other_configs"]))
    if "diloco_outer_step" in d:
        out.append("  diloco_outer_step: " + json.dumps({k: v for k, v in d["diloco_outer_step"].items() if k != "workload"}))
    return "\n".join(out)


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("kind", choices=("trace", "traffic", "counters"))
    ap.add_argument("dirs", nargs="+")
    ap.add_argument("--title", default="")
    ap.add_argument("--command", action="append", default=[])
    ap.add_argument("--note", action="append", default=[])
    ap.add_argument("--bench-json", default="", help="stdout of the profiled bench.py run: its own figures are appended")
    args = ap.parse_args(argv)
    head = []
    if args.title:
        head.append(args.title)
    for c in args.command:
        head.append("command: " + c)
    head.append("device: AMD Instinct MI355X (gfx950, 256 CUs), ROCm 7.2; durations in microseconds; torch's own kernels omitted")
    head.append("")
    if args.kind == "trace":
        body = trace(args.dirs[0])
    elif args.kind == "traffic":
        if len(args.dirs) != 2:
            raise SystemExit("traffic needs the FETCH_SIZE directory and the WRITE_SIZE directory")
        body = traffic(args.dirs[0], args.dirs[1])
    else:
        body = counters(args.dirs)
    tail = bench_excerpt(args.bench_json) if args.bench_json else ""
    notes = "".join("\nnote: " + n for n in args.note)
    print("\n".join(head) + body + ("\n" + tail if tail else "") + notes)
    return 0


if __name__ == "__main__":
    sys.exit(main())
