#!/usr/bin/env python3
"""Per-kernel means of the counters of one or more `rocprofv3 --pmc ... --output-format csv` runs.

    python3 gemm-zoo_amd/bench/pmc_table.py gpurun_out/pmc_a gpurun_out/pmc_b [--skip fill,elementwise]

Every directory is searched for *counter_collection.csv; one line per (kernel, counter): mean over the dispatches
of that kernel, and the number of dispatches.  Text in, text out: what goes into profiles/ is this output.
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
            print(f"    {c:40s} {sum(vals) / len(vals):18,.0f}   ({len(vals)} dispatches)")
    return 0


if __name__ == "__main__":
    sys.exit(main())
