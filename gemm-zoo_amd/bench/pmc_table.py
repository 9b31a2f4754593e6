#!/usr/bin/env python3
"""Per-kernel means of the counters of one or more `rocprofv3 --pmc ... --output-format csv` runs.

    python3 gemm-zoo_amd/bench/pmc_table.py out/pmc_a out/pmc_b [--skip fill,elementwise]

Every directory is searched for *counter_collection.csv; one line per (kernel, counter): mean, minimum and maximum
over the dispatches of that kernel, and their number.  With --levels the dispatches of a kernel are also grouped by
value (groups of values within 2 % of each other): a kernel that ran two workloads in one process - with and without
reading C, a small copy and a large one - shows one line per workload.  Text in, text out: what goes into profiles/
is this output.
"""
import argparse
import collections
import csv
import pathlib
import sys


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("dirs", nargs="+")
    ap.add_argument("--skip", default="fill_kernel,elementwise,compare", help="kernel-name substrings to leave out")
    ap.add_argument("--width", type=int, default=96)
    ap.add_argument("--levels", action="store_true", help="also list the groups of near-equal values per counter")
    args = ap.parse_args()
    skip = [s for s in args.skip.split(",") if s]
    table = collections.OrderedDict()
    for d in args.dirs:
        for f in sorted(pathlib.Path(d).rglob("*counter_collection.csv")):
            with open(f, newline="") as fh:
                for r in csv.DictReader(fh):
                    name = r["Kernel_Name"]
                    if any(s in name for s in skip):
                        continue
                    table.setdefault(name, collections.OrderedDict()).setdefault(r["Counter_Name"], []).append(
                        float(r["Counter_Value"]))
    for name, counters in table.items():
        print(name[:args.width])
        for c, vals in counters.items():
            print(f"    {c:40s} {sum(vals) / len(vals):18,.0f}   min {min(vals):,.0f}  max {max(vals):,.0f}  ({len(vals)} dispatches)")
            if args.levels and max(vals) > 1.02 * min(vals):
                groups = []
                for v in sorted(vals):
                    if groups and v <= 1.02 * groups[-1][0]:
                        groups[-1].append(v)
                    else:
                        groups.append([v])
                for g in groups:
                    print(f"        level {sum(g) / len(g):18,.1f}   x {len(g)}")
    return 0


if __name__ == "__main__":
    sys.exit(main())
