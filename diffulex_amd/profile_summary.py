"""Turn rocprofv3 output of ``bench.py`` runs into the short summaries kept under ``profiles/``.

    python -m diffulex_amd.profile_summary --workload c3 --dir prof_c3 [--write-traffic]

``--dir`` holds what these commands wrote (each in a run of its own; W = the workload):

    rocprofv3 --kernel-trace --stats --output-format csv -d DIR/kt -o r -- python3 bench.py --workload W --no-cpu
    rocprofv3 --pmc FETCH_SIZE --kernel-trace --output-format csv -d DIR/FETCH_SIZE -o r -- python3 bench.py --workload W --steps 8 --warmup 2 --no-cpu
    rocprofv3 --pmc WRITE_SIZE --kernel-trace --output-format csv -d DIR/WRITE_SIZE -o r -- python3 bench.py --workload W --steps 8 --warmup 2 --no-cpu
    rocprofv3 --pmc FETCH_SIZE --kernel-trace --output-format csv -d DIR/cal_FETCH_SIZE -o r -- python3 bench.py --calibrate-copy --steps 4
    rocprofv3 --pmc WRITE_SIZE --kernel-trace --output-format csv -d DIR/cal_WRITE_SIZE -o r -- python3 bench.py --calibrate-copy --steps 4

and, optionally, ``DIR/bench.json`` with the JSON line of the kernel-trace run.  The counters are
in KiB per dispatch; they are scaled by what the same counter reads for a plain device copy of
1 GiB (1 GiB read, 1 GiB written).  Prints a Markdown summary; ``--write-traffic`` also records
the HBM bytes per launch of the attention kernel in ``profiles/traffic.json``, where ``bench.py``
reads its ``roofline.traffic`` from.
"""
from __future__ import annotations

import argparse
import collections
import csv
import glob
import json
import os

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
GIB = 1 << 30


def short(name: str) -> str:
    name = name.replace("(anonymous namespace)::", "")
    return name.split("(")[0].replace("void dfx::", "").replace("void ", "")[-90:]


def kernel_stats(d):
    rows = []
    for fn in glob.glob(os.path.join(d, "kt", "**", "*kernel_stats.csv"), recursive=True):
        for r in csv.DictReader(open(fn)):
            rows.append((short(r["Name"]), int(r["Calls"]), float(r["AverageNs"]) / 1e3, float(r["MinNs"]) / 1e3,
                         float(r["MaxNs"]) / 1e3, float(r["Percentage"])))
    return sorted(rows, key=lambda r: -r[5])


def counter_per_dispatch(d, sub):
    total, count = collections.defaultdict(float), collections.Counter()
    for fn in glob.glob(os.path.join(d, sub, "**", "*counter_collection.csv"), recursive=True):
        for r in csv.DictReader(open(fn)):
            k = short(r["Kernel_Name"])
            total[k] += float(r["Counter_Value"])
            count[k] += 1
    return {k: (total[k] / count[k], count[k]) for k in total}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--workload", required=True)
    ap.add_argument("--dir", required=True)
    ap.add_argument("--kernel", default="paged_attn", help="substring naming the kernel whose traffic is recorded")
    ap.add_argument("--write-traffic", action="store_true")
    ap.add_argument("--counters", nargs="*", default=[],
                    help="sub-directories of --dir holding other `rocprofv3 --pmc ...` runs of the same command: their "
                         "counters are listed as means per dispatch of the kernel named by --kernel")
    args = ap.parse_args()
    if args.counters:
        print(f"## counters of `{args.kernel}` kernels, workload {args.workload} (mean per dispatch, summed over the chip)\n")
        print("| counter | kernel | mean per dispatch | dispatches |")
        print("|---|---|---|---|")
        for sub in args.counters:
            total, count = collections.defaultdict(float), collections.Counter()
            for fn in glob.glob(os.path.join(args.dir, sub, "**", "*counter_collection.csv"), recursive=True):
                for r in csv.DictReader(open(fn)):
                    k = short(r["Kernel_Name"])
                    if args.kernel in k and "plan" not in k:
                        total[(r["Counter_Name"], k)] += float(r["Counter_Value"])
                        count[(r["Counter_Name"], k)] += 1
            for (c, k) in sorted(total):
                print(f"| `{c}` | `{k}` | {total[(c, k)] / count[(c, k)]:,.0f} | {count[(c, k)]} |")
        return

    bench = None
    path = os.path.join(args.dir, "bench.json")
    if os.path.exists(path):
        for line in open(path):
            if line.startswith("{"):
                bench = json.loads(line)
    print(f"## kernel trace, workload {args.workload}\n")
    print("| kernel | calls | avg us | min us | max us | % of GPU time |")
    print("|---|---|---|---|---|---|")
    for name, calls, avg, lo, hi, pct in kernel_stats(args.dir):
        print(f"| `{name}` | {calls} | {avg:.2f} | {lo:.2f} | {hi:.2f} | {pct:.1f} |")
    if bench is not None:
        print(f"\nbench.py of the same run: ms_per_step {bench['ms_per_step']:.5f}, roofline.frac "
              f"{bench['roofline']['frac']:.4f}, config {json.dumps(bench['config'])}")

    factors = {}
    for c in ("FETCH_SIZE", "WRITE_SIZE"):
        cal = counter_per_dispatch(args.dir, "cal_" + c)
        if cal:
            # the copy moves 1 GiB each way; nothing else in that run moves more (its source is
            # filled by a kernel that writes 1 GiB and reads nothing)
            kib = max(v[0] for v in cal.values())
            factors[c] = GIB / (kib * 1024.0)
    if not factors:
        return
    print("\n## HBM traffic per dispatch (KiB counters scaled by a 1 GiB device copy)\n")
    print("| kernel | FETCH_SIZE KiB | WRITE_SIZE KiB | scaled bytes read | scaled bytes written |")
    print("|---|---|---|---|---|")
    fetch = counter_per_dispatch(args.dir, "FETCH_SIZE")
    write = counter_per_dispatch(args.dir, "WRITE_SIZE")
    chosen = None
    for k in sorted(set(fetch) | set(write)):
        f, w = fetch.get(k, (0.0, 0))[0], write.get(k, (0.0, 0))[0]
        rb, wb = f * 1024 * factors.get("FETCH_SIZE", 1.0), w * 1024 * factors.get("WRITE_SIZE", 1.0)
        print(f"| `{k}` | {f:.1f} | {w:.1f} | {rb / 1e6:.2f} MB | {wb / 1e6:.2f} MB |")
        if args.kernel in k and "plan" not in k and (chosen is None or rb + wb > chosen[1] + chosen[2]):
            chosen = (k, rb, wb)
    print(f"\nscale factors: FETCH_SIZE x{factors.get('FETCH_SIZE', float('nan')):.4f}, "
          f"WRITE_SIZE x{factors.get('WRITE_SIZE', float('nan')):.4f}")
    if chosen is None:
        return
    k, rb, wb = chosen
    alg = bench["roofline"].get("algorithmic_bytes") if bench else None
    print(f"\n`{k}`: {(rb + wb) / 1e6:.1f} MB per launch" + (f" = {(rb + wb) / alg:.3f} x the algorithmic {alg / 1e6:.1f} MB" if alg else ""))
    if args.write_traffic and alg:
        out = os.path.join(ROOT, "profiles", "traffic.json")
        data = {}
        if os.path.exists(out):
            data = json.load(open(out))
        data[args.workload] = {"bytes": round(rb + wb), "read_bytes": round(rb), "written_bytes": round(wb),
                               "algorithmic_bytes": int(alg), "kernel": k,
                               "source": f"rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE of `python3 bench.py --workload {args.workload} "
                                         "--steps 8 --warmup 2 --no-cpu`, scaled by a 1 GiB device copy"}
        json.dump(data, open(out, "w"), indent=1, sort_keys=True)
        print(f"\nrecorded in profiles/traffic.json")


if __name__ == "__main__":
    main()
