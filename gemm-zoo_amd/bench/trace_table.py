#!/usr/bin/env python3
"""Per-kernel durations of a `rocprofv3 --kernel-trace --output-format csv` run, leg by leg.

    python3 gemm-zoo_amd/bench/trace_table.py out/prof_stats [--min-run 100] [--window 200:800]

A process like bench.py launches the same kernel for several workloads one after the other (beta = 0, then
alpha = beta = 1).  The dispatches of a kernel are therefore cut into RUNS - maximal sequences in start order that no
dispatch of another kernel interrupts (fills, compares and copies excepted: --ignore) - and every run of at least
--min-run dispatches gets a line of its own: count, mean, minimum and maximum duration in microseconds.  --window
A:B adds the mean over the dispatches [len - B, len - A) of each run, counted from its end: with bench.py's default
flags the last 200 launches of a leg carry an event pair each and the 600 before them are the timed blocks, so
--window 200:800 is the profiler's figure for exactly the launches behind `kernel_ms_mean`.
"""
import argparse
import csv
import pathlib
import sys


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("dirs", nargs="+")
    ap.add_argument("--min-run", type=int, default=100)
    ap.add_argument("--window", default="", help="A:B, dispatches counted from the end of a run")
    ap.add_argument("--ignore", default="fill_kernel,compare_kernel,__amd_rocclr", help="kernels that do not end a run")
    ap.add_argument("--width", type=int, default=100)
    args = ap.parse_args()
    ignore = [s for s in args.ignore.split(",") if s]
    rows = []
    for d in args.dirs:
        for f in sorted(pathlib.Path(d).rglob("*kernel_trace.csv")):
            with open(f, newline="") as fh:
                for r in csv.DictReader(fh):
                    rows.append((int(r["Start_Timestamp"]), int(r["End_Timestamp"]), r["Kernel_Name"]))
    rows.sort()
    runs = []   # (name, [durations in us])
    for start, end, name in rows:
        if any(s in name for s in ignore):
            continue
        if not runs or runs[-1][0] != name:
            runs.append((name, []))
        runs[-1][1].append((end - start) / 1e3)
    lo = hi = None
    if args.window:
        lo, hi = (int(x) for x in args.window.split(":"))
    for name, us in runs:
        if len(us) < args.min_run:
            continue
        line = f"{name[:args.width]:{args.width}s} {len(us):6d}  mean {sum(us) / len(us):9.2f}  min {min(us):9.2f}  max {max(us):9.2f}"
        if hi is not None and len(us) >= hi:
            w = us[len(us) - hi:len(us) - lo]
            line += f"   window [-{hi}, -{lo}): mean {sum(w) / len(w):9.2f} over {len(w)}"
        print(line)
    return 0


if __name__ == "__main__":
    sys.exit(main())
