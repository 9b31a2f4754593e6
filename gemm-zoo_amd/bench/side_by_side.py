#!/usr/bin/env python3
"""This library's kernel and hipBLASLt's on the same operands in ONE process, for timing and for counter runs.

The reference times cuBLASLt beside its own kernels (nvidia/utils/cublaslt_gemm.cuh:52-129); this driver does the
same per problem and is what the `rocprofv3 --pmc` runs under profiles/ execute, so that both kernels see the same
machine, the same clocks and the same operands:

    python3 gemm-zoo_amd/bench/side_by_side.py --types bf16bf16bf16 --m 4096 --n 4096 --k 4096,8192
    rocprofv3 --pmc SQ_INSTS_LDS SQ_INSTS_VALU ... -- python3 gemm-zoo_amd/bench/side_by_side.py --launches 6 --no-timing

With --no-timing the kernels run alternately, `--launches` times each (what a counter run wants: every dispatch is
serialised by the profiler anyway).  Otherwise each side is timed in blocks of back-to-back launches over rotating
operand sets after a settling phase, the two sides alternating block by block, with HIP events around each block.
"""
import argparse
import importlib
import json
import pathlib
import sys
import time

ROOT = pathlib.Path(__file__).resolve().parents[2]
sys.path.insert(0, str(ROOT))


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--types", default="bf16bf16f32")
    ap.add_argument("--m", type=int, default=4096)
    ap.add_argument("--n", type=int, default=4096)
    ap.add_argument("--k", default="4096", help="comma-separated list")
    ap.add_argument("--layout-a", default="row", choices=["row", "col"])
    ap.add_argument("--layout-b", default="col", choices=["row", "col"])
    ap.add_argument("--variants", default="0", help="comma-separated MFMA-rung variants of this library (0 = launcher)")
    ap.add_argument("--beta", type=float, default=0.0)
    ap.add_argument("--launches", type=int, default=100, help="launches per timed block (or per side with --no-timing)")
    ap.add_argument("--blocks", type=int, default=3)
    ap.add_argument("--sets", type=int, default=0, help="rotating operand sets (0: enough to exceed 256 MB)")
    ap.add_argument("--settle", type=float, default=0.3, help="seconds of back-to-back launches before timing")
    ap.add_argument("--no-timing", action="store_true")
    ap.add_argument("--no-vendor", action="store_true")
    args = ap.parse_args()

    import torch

    capi = importlib.import_module("gemm-zoo_amd.capi")
    functors = importlib.import_module("gemm-zoo_amd.functors")
    if not torch.cuda.is_available():
        print("side_by_side.py: no GPU visible", file=sys.stderr)
        return 3
    types = {name: t for t, name in capi.TYPES_NAMES.items()}[args.types]
    tin = {1: torch.int8, 2: torch.bfloat16, 4: torch.float32}[capi.IN_SIZE[types]]
    if types == capi.F16F16F16:
        tin = torch.float16
    if types in (capi.E4M3E4M3F16, capi.E5M2E5M2F16):
        tin = torch.float8_e4m3fn if types == capi.E4M3E4M3F16 else torch.float8_e5m2
    tout = {capi.S8S8S32: torch.int32, capi.BF16BF16F32: torch.float32, capi.BF16BF16BF16: torch.bfloat16,
            capi.F32F32F32: torch.float32}.get(types, torch.float16)
    in_dt = {capi.S8S8S32: capi.DT_INT8, capi.BF16BF16F32: capi.DT_BF16, capi.BF16BF16BF16: capi.DT_BF16,
             capi.F16F16F16: capi.DT_F16, capi.F32F32F32: capi.DT_F32, capi.E4M3E4M3F16: capi.DT_E4M3,
             capi.E5M2E5M2F16: capi.DT_E5M2}[types]
    out_dt = {capi.S8S8S32: capi.DT_INT32, capi.BF16BF16F32: capi.DT_F32, capi.BF16BF16BF16: capi.DT_BF16,
              capi.F32F32F32: capi.DT_F32}.get(types, capi.DT_F16)
    la = capi.ROW_MAJOR if args.layout_a == "row" else capi.COL_MAJOR
    lb = capi.ROW_MAJOR if args.layout_b == "row" else capi.COL_MAJOR
    dev = torch.device("cuda:0")
    stream = torch.cuda.current_stream()
    sptr = stream.cuda_stream
    m, n = args.m, args.n
    kind = capi.FILL_INT8_UNIFORM if types == capi.S8S8S32 else capi.FILL_NORMAL
    scale_b = 0.25 if capi.IN_SIZE[types] == 1 and types != capi.S8S8S32 else 1.0
    variants = [int(v) for v in args.variants.split(",")]
    rows = []
    for k in [int(x) for x in args.k.split(",")]:
        ab_bytes = capi.IN_SIZE[types] * (m * k + k * n)
        nsets = args.sets or (256 * 1000 * 1000 + capi.OUT_SIZE[types] * m * n) // ab_bytes + 2
        sets = []
        for j in range(nsets):
            a = torch.empty(m * k, dtype=tin, device=dev)
            b = torch.empty(k * n, dtype=tin, device=dev)
            capi.fill(a, m * k, in_dt, kind, 1.0, 2025 + 3 * j, sptr)
            capi.fill(b, k * n, in_dt, kind, scale_b, 2026 + 3 * j, sptr)
            sets.append((a, b))
        d = torch.empty(m * n, dtype=tout, device=dev)
        c = None
        if args.beta:
            c = torch.empty(m * n, dtype=tout, device=dev)
            capi.fill(c, m * n, out_dt, kind, 1.0, 4242, sptr)
        sides = {}
        for v in variants:
            def ours(i, v=v):
                a, b = sets[i % nsets]
                capi.gemm(types, a, b, c, d, m, n, k, la, lb, 1, args.beta, capi.RUNG_MFMA, v, sptr)
            sides[f"ours_v{v}"] = ours
        lt = None
        if not args.no_vendor:
            lt = functors.HipblasLtGemm(types, m, n, k, la, lb)

            def theirs(i):
                a, b = sets[i % nsets]
                lt(a, b, c, d, 1, args.beta, stream)
            sides["hipblaslt"] = theirs
        it = 0
        if args.no_timing:
            for _ in range(args.launches):
                for fn in sides.values():
                    fn(it)
                    it += 1
            torch.cuda.synchronize()
            rows.append({"k": k, "launches_per_side": args.launches})
        else:
            t0 = time.perf_counter()
            while time.perf_counter() - t0 < args.settle:
                for fn in sides.values():
                    for _ in range(16):
                        fn(it)
                        it += 1
                torch.cuda.synchronize()
            res = {name: [] for name in sides}
            for _ in range(args.blocks):
                for name, fn in sides.items():
                    for _ in range(20):   # this side's own clock state before its block
                        fn(it)
                        it += 1
                    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                    e0.record(stream)
                    for _ in range(args.launches):
                        fn(it)
                        it += 1
                    e1.record(stream)
                    e1.synchronize()
                    res[name].append(e0.elapsed_time(e1) / args.launches * 1e3)
            row = {"k": k, "sets": nsets}
            for name, us in res.items():
                row[name + "_us"] = [round(x, 2) for x in us]
            rows.append(row)
            print(f"{args.types} {m}x{n}x{k} {args.layout_a}/{args.layout_b} beta={args.beta}: " +
                  "  ".join(f"{name} {min(us):.2f} us (" + " ".join(f"{x:.1f}" for x in us) + ")"
                            for name, us in res.items()), flush=True)
        if lt is not None:
            lt.close()
        del sets, d, c
    print(json.dumps({"types": args.types, "m": m, "n": n, "layout_a": args.layout_a, "layout_b": args.layout_b,
                      "beta": args.beta, "rows": rows}))
    return 0


if __name__ == "__main__":
    sys.exit(main())
