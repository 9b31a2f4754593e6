#!/usr/bin/env python3
"""Every rung of the ladder on ONE problem, timed with HIP events, one result line per rung.

The reference has one bench main per rung (nvidia/bench/bench_{naive,tiling_*,rmem_*,double_buffered_*,
async_buffered_*,bf16_mma_gemm}.cu); this runs them back to back on the same operands so that a hardware-counter run
of this command (rocprofv3 --pmc ...) shows, kernel by kernel, what each step of the ladder bought.

    python3 gemm-zoo_amd/bench/ladder.py --types bf16bf16f32 --size 4096 --layout-b col

Rungs 0-3 add the products of one output in k order, so the first rung's output is the reference for the others:
bit-exact for rungs 1-3 on any data; the MFMA rung is checked with the tolerance of its type.
"""
import argparse
import importlib
import json
import pathlib
import sys

ROOT = pathlib.Path(__file__).resolve().parents[2]
sys.path.insert(0, str(ROOT))


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--types", default="bf16bf16f32",
                    choices=["s8s8s32", "bf16bf16f32", "bf16bf16bf16", "f16f16f16", "f32f32f32", "e4m3e4m3f16", "e5m2e5m2f16",
                             "bf16bf16bf16_acc16", "f16f16f16_acc16"])
    ap.add_argument("--size", type=int, default=4096, help="M = N = K")
    ap.add_argument("--layout-a", default="row", choices=["row", "col"])
    ap.add_argument("--layout-b", default="col", choices=["row", "col"])
    ap.add_argument("--reps", type=int, default=5, help="timed launches per rung (the two slowest rungs run once)")
    ap.add_argument("--fill", default="default", choices=["default", "small-int"],
                    help="default: N(0,1) for floats, uniform int8 for s8; small-int: values in {-1,0,1}")
    args = ap.parse_args()

    import torch

    capi = importlib.import_module("gemm-zoo_amd.capi")  # raises if the HIP library is not built
    if not torch.cuda.is_available():
        print("ladder.py: no GPU visible", file=sys.stderr)
        return 3
    types = {name: t for t, name in capi.TYPES_NAMES.items()}[args.types]
    f8 = (capi.E4M3E4M3F16, capi.E5M2E5M2F16)
    tin = {capi.S8S8S32: torch.int8, capi.BF16BF16F32: torch.bfloat16, capi.BF16BF16BF16: torch.bfloat16,
           capi.F16F16F16: torch.float16, capi.F32F32F32: torch.float32, capi.E4M3E4M3F16: torch.float8_e4m3fn,
           capi.E5M2E5M2F16: torch.float8_e5m2, capi.BF16BF16BF16_ACC16: torch.bfloat16,
           capi.F16F16F16_ACC16: torch.float16}[types]
    tout = {capi.S8S8S32: torch.int32, capi.BF16BF16F32: torch.float32, capi.BF16BF16BF16: torch.bfloat16,
            capi.BF16BF16BF16_ACC16: torch.bfloat16, capi.F32F32F32: torch.float32}.get(types, torch.float16)
    in_dt = {capi.S8S8S32: capi.DT_INT8, capi.BF16BF16F32: capi.DT_BF16, capi.BF16BF16BF16: capi.DT_BF16,
             capi.F16F16F16: capi.DT_F16, capi.F32F32F32: capi.DT_F32, capi.E4M3E4M3F16: capi.DT_E4M3,
             capi.E5M2E5M2F16: capi.DT_E5M2, capi.BF16BF16BF16_ACC16: capi.DT_BF16,
             capi.F16F16F16_ACC16: capi.DT_F16}[types]
    out_dt = {capi.S8S8S32: capi.DT_INT32, capi.BF16BF16F32: capi.DT_F32, capi.BF16BF16BF16: capi.DT_BF16,
              capi.BF16BF16BF16_ACC16: capi.DT_BF16, capi.F32F32F32: capi.DT_F32}.get(types, capi.DT_F16)
    la = capi.ROW_MAJOR if args.layout_a == "row" else capi.COL_MAJOR
    lb = capi.ROW_MAJOR if args.layout_b == "row" else capi.COL_MAJOR
    n = args.size
    dev = torch.device("cuda:0")
    sptr = torch.cuda.current_stream().cuda_stream

    a = torch.empty(n * n, dtype=tin, device=dev)
    b = torch.empty(n * n, dtype=tin, device=dev)
    if args.fill == "small-int":
        kind = capi.FILL_SMALL_INT
    else:
        kind = capi.FILL_INT8_UNIFORM if types == capi.S8S8S32 else capi.FILL_NORMAL
    # 8-bit float inputs, fp16 output: B ~ N(0, 1/16) keeps sums over K far from the fp16 range
    capi.fill(a, n * n, in_dt, kind, 1.0, 2025, sptr)
    capi.fill(b, n * n, in_dt, kind, 0.25 if types in f8 and args.fill == "default" else 1.0, 2026, sptr)
    ref = torch.empty(n * n, dtype=tout, device=dev)
    d = torch.empty(n * n, dtype=tout, device=dev)

    rungs = [capi.RUNG_NAIVE, capi.RUNG_COALESCED, capi.RUNG_LDS_TILED, capi.RUNG_DOUBLE_BUFFERED, capi.RUNG_MFMA]
    flops = 2.0 * n * n * n
    rows = []
    for rung in rungs:
        out = ref if rung == capi.RUNG_NAIVE else d
        reps = 1 if rung in (capi.RUNG_NAIVE, capi.RUNG_COALESCED) else args.reps
        capi.gemm(types, a, b, None, out, n, n, n, la, lb, 1.0, 0.0, rung, 0, sptr)  # warm-up, result kept
        torch.cuda.synchronize()
        times = []
        for _ in range(reps):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            capi.gemm(types, a, b, None, out, n, n, n, la, lb, 1.0, 0.0, rung, 0, sptr)
            e1.record()
            e1.synchronize()
            times.append(e0.elapsed_time(e1))
        ms = sum(times) / len(times)
        if rung == capi.RUNG_NAIVE:
            bad = 0
        elif rung != capi.RUNG_MFMA or types == capi.S8S8S32:
            bad = capi.compare(d, ref, n * n, out_dt, 0.0, sptr)
        else:  # another summation order: |x - ref| <= tol * (sqrt(k) + |ref|)
            tol = 1e-3 if types == capi.BF16BF16F32 else 1e-4 if types == capi.F32F32F32 else 1e-2
            bad = capi.compare(d, ref, n * n, out_dt, tol * n ** 0.5, sptr, rel_threshold=tol)
        p = capi.plan(types, n, n, n, la, lb, rung, 0)
        row = {"rung": capi.rung_name(rung), "ms": round(ms, 4), "tflops": round(flops / ms / 1e9, 2),
               "tile": [p.tile_m, p.tile_n, p.tile_k], "threads": p.threads, "lds_bytes": p.lds_bytes,
               "different_from_rung0": int(bad)}
        rows.append(row)
        print(f"{row['rung']:>16s}  {ms:10.4f} ms  {row['tflops']:9.2f} T  tile {p.tile_m}x{p.tile_n}x{p.tile_k}  "
              f"mismatches {bad}", flush=True)
    print(json.dumps({"types": args.types, "size": n, "layout_a": args.layout_a, "layout_b": args.layout_b,
                      "fill": args.fill, "rungs": rows}))
    return 1 if any(r["different_from_rung0"] for r in rows) else 0


if __name__ == "__main__":
    sys.exit(main())
