#!/usr/bin/env python3
"""Headline benchmark: bf16 x bf16 -> f32 GEMM, M=N=K=4096, A row-major, B column-major, on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-extras] [--no-cpu-baseline]

One "step" is one launch of the GEMM on one of P rotating input sets that are already
resident in HBM (P is sized on the bytes that rotate, A and B, so that the 256 MB Infinity
Cache cannot hold them between launches).  Prints ONE JSON line.

What is timed does not depend on the flags: after the W warm-up launches the same launches go
on until the part's clocks have settled (SETTLE_SECONDS of back-to-back launches: the matrix
cores run against a power limit and the clock takes tens of milliseconds to come down to what
the kernel sustains).  Then blocks of K launches are timed back to back, as many blocks as it
takes to fill MIN_TIMED_SECONDS; `ms_per_step` and `value` are the mean over all of them.
`roofline.achieved` uses HIP events recorded on the launch stream before and after each of those
blocks: the kernels' own time over the same launches (it agrees with the rocprofv3 kernel trace of
such a run to a fraction of a percent; an event pair around every single launch, also reported,
adds about 5 us per launch).

Beside it the line carries the int8 8192^3 and the skinny (decode) shapes, the hipBLASLt
comparator when its library is built, and the CPU restatement of the reference GEMM timed
on this machine's host cores on a bounded sample.
"""
from __future__ import annotations

import argparse
import importlib
import json
import os
import sys
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
sys.path.insert(0, str(ROOT))

PEAK_TFLOPS = {"bf16": 2500.0, "f16": 2500.0, "s8": 5000.0, "fp8": 5000.0, "f32": 157.3}  # dense MFMA, MI355X
PEAK_HBM_GBS = 8000.0
INFINITY_CACHE_BYTES = 256 * 1000 * 1000
SETTLE_SECONDS = 0.3       # back-to-back launches before anything is timed, whatever --warmup says
MIN_TIMED_SECONDS = 0.05   # the timed region is at least this long: blocks of --steps launches are repeated
EVENT_LAUNCHES = 200       # single launches timed with an event pair each


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=300,
                    help="untimed launches first; the matrix-core clock takes tens of milliseconds to settle")
    ap.add_argument("--no-extras", action="store_true", help="skip the s8 8192^3 and skinny side measurements")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--cpu-seconds", type=float, default=12.0, help="target CPU time of the baseline sample")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also launch one plain 256 MiB device copy (known traffic) so that a counter run of this "
                         "command holds the scale for FETCH_SIZE / WRITE_SIZE")
    args = ap.parse_args()

    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build measures ONE GPU (the GEMM path has no cross-GPU exchange; "
              "shard N or M across GPUs and run the same kernel per shard). Use --gpus 1.", file=sys.stderr)
        return 2

    import torch

    capi = importlib.import_module("gemm-zoo_amd.capi")  # raises if the HIP library is not built
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        return 3
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    stream = torch.cuda.current_stream()
    sptr = stream.cuda_stream

    IN_T = {capi.S8S8S32: torch.int8, capi.BF16BF16F32: torch.bfloat16, capi.BF16BF16BF16: torch.bfloat16,
            capi.F16F16F16: torch.float16, capi.E4M3E4M3F16: torch.float8_e4m3fn, capi.E5M2E5M2F16: torch.float8_e5m2,
            capi.F32F32F32: torch.float32}
    OUT_T = {capi.S8S8S32: torch.int32, capi.BF16BF16F32: torch.float32, capi.BF16BF16BF16: torch.bfloat16,
             capi.F16F16F16: torch.float16, capi.E4M3E4M3F16: torch.float16, capi.E5M2E5M2F16: torch.float16,
             capi.F32F32F32: torch.float32}
    OUT_DT = {capi.S8S8S32: capi.DT_INT32, capi.BF16BF16F32: capi.DT_F32, capi.BF16BF16BF16: capi.DT_BF16,
              capi.F16F16F16: capi.DT_F16, capi.E4M3E4M3F16: capi.DT_F16, capi.E5M2E5M2F16: capi.DT_F16,
              capi.F32F32F32: capi.DT_F32}
    IN_DT = {capi.S8S8S32: capi.DT_INT8, capi.BF16BF16F32: capi.DT_BF16, capi.BF16BF16BF16: capi.DT_BF16,
             capi.F16F16F16: capi.DT_F16, capi.E4M3E4M3F16: capi.DT_E4M3, capi.E5M2E5M2F16: capi.DT_E5M2,
             capi.F32F32F32: capi.DT_F32}

    def make_sets(types, m, n, k, scale_b=1.0, seed0=2025, c_bytes=0):
        """P rotating (A, B) sets + one D, filled on the device (seeds 2025, 2026, ... as the reference harness).
        P counts the bytes that rotate: one pass over all sets must push D (and C) plus a cache full of operands
        through the Infinity Cache, so that no launch finds its operands there."""
        es = capi.IN_SIZE[types]
        ab_bytes = es * (m * k + k * n)
        d_bytes = capi.OUT_SIZE[types] * m * n
        p = -(-(INFINITY_CACHE_BYTES + d_bytes + c_bytes) // ab_bytes) + 1
        kind = capi.FILL_INT8_UNIFORM if types == capi.S8S8S32 else capi.FILL_NORMAL
        sets = []
        for j in range(p):
            a = torch.empty(m * k, dtype=IN_T[types], device=dev)
            b = torch.empty(k * n, dtype=IN_T[types], device=dev)
            capi.fill(a, m * k, IN_DT[types], kind, 1.0, seed0 + 3 * j, sptr)
            capi.fill(b, k * n, IN_DT[types], kind, scale_b, seed0 + 3 * j + 1, sptr)
            sets.append((a, b))
        d = torch.empty(m * n, dtype=OUT_T[types], device=dev)
        return sets, d, ab_bytes + d_bytes

    def timed(types, m, n, k, la, lb, steps, warmup, rung=capi.RUNG_AUTO, variant=0, scale_b=1.0, verify=True,
              vendor=None, beta=0):
        c_bytes = capi.OUT_SIZE[types] * m * n if beta else 0
        sets, d, problem_bytes = make_sets(types, m, n, k, scale_b, c_bytes=c_bytes)
        p = len(sets)
        c = None
        if beta:  # the reference's drivers run alpha = beta = 1 (nvidia/bench/bench_bf16_mma_gemm.cu:15-16)
            c = torch.empty(m * n, dtype=OUT_T[types], device=dev)
            capi.fill(c, m * n, OUT_DT[types], capi.FILL_INT8_UNIFORM if types == capi.S8S8S32 else capi.FILL_NORMAL, 1.0, 4242,
                      sptr)
            problem_bytes += c_bytes

        def launch(i):
            a, b = sets[i % p]
            if vendor is not None:  # the comparator library on the same operands
                vendor(a, b, c, d, 1, beta, stream)
            else:
                capi.gemm(types, a, b, c, d, m, n, k, la, lb, 1, beta, rung, variant, sptr)

        if verify:  # verify-once, against an independent rung of the ladder (sequential-k LDS kernel)
            launch(0)
            ref = torch.empty_like(d)
            a, b = sets[0]
            capi.gemm(types, a, b, c, ref, m, n, k, la, lb, 1, beta, capi.RUNG_LDS_TILED, 0, sptr)
            if types == capi.S8S8S32:
                ndiff = capi.compare(d, ref, m * n, capi.DT_INT32, 0.0, sptr)
            else:
                dt = OUT_DT[types]
                # sanity bound only (parity proper lives in tests/): fp32 accumulation in a different order, so allow
                # 1e-3 of the output scale for fp32 out and one 16-bit ulp at 4 sigma for 16-bit out
                scale = float(torch.sqrt(torch.tensor(float(k)))) * scale_b
                tol = (1e-3 if types in (capi.BF16BF16F32, capi.F32F32F32) else 4e-2) * scale
                ndiff = capi.compare(d, ref, m * n, dt, tol, sptr)
            if ndiff:
                raise RuntimeError(f"verification failed: {ndiff} elements differ ({capi.TYPES_NAMES[types]} {m}x{n}x{k})")
            del ref
        it = 0
        for _ in range(warmup):
            launch(it)
            it += 1
        # clock settle, by time: the same launches back to back, in batches that keep the queue full
        torch.cuda.synchronize()
        t_settle = time.perf_counter()
        settle_launches = 0
        while time.perf_counter() - t_settle < SETTLE_SECONDS:
            for _ in range(32):
                launch(it)
                it += 1
            settle_launches += 32
            torch.cuda.synchronize()
        # the timed region: blocks of exactly `steps` launches back to back, nothing else on the stream but one HIP
        # event before and after each block (torch events on torch's current stream, which is the stream the launches
        # go to): the events give the kernels' own time, the host clock around the same block the wall time
        blocks, wall, pairs = 0, 0.0, []
        while blocks == 0 or wall < MIN_TIMED_SECONDS:
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            e0.record(stream)
            for _ in range(steps):
                launch(it)
                it += 1
            e1.record(stream)
            torch.cuda.synchronize()
            wall += time.perf_counter() - t0
            pairs.append((e0, e1))
            blocks += 1
        launches = blocks * steps
        kernel_ms = sum(a.elapsed_time(b) for a, b in pairs) / launches
        # for comparison: single launches of the same sequence with an event pair around each.  The pair itself costs
        # about 5 us on the stream (kernel trace of the same launches: 100.8 us where the pairs say 105.9), so this
        # figure is reported but not used.
        nev = EVENT_LAUNCHES
        starts = [torch.cuda.Event(enable_timing=True) for _ in range(nev)]
        stops = [torch.cuda.Event(enable_timing=True) for _ in range(nev)]
        for i in range(nev):
            starts[i].record(stream)
            launch(it)
            it += 1
            stops[i].record(stream)
        torch.cuda.synchronize()
        ev = sorted(s.elapsed_time(e) for s, e in zip(starts, stops))
        wall_ms = wall * 1e3 / launches
        return {"wall_ms": wall_ms, "kernel_ms_mean": kernel_ms, "single_launch_ms_mean": sum(ev) / len(ev),
                "single_launch_ms_median": ev[len(ev) // 2], "problem_bytes": problem_bytes, "sets": p,
                "timed_blocks": blocks, "settle_launches": settle_launches, "event_launches": nev}

    if args.copy_calibration:
        src = torch.empty(256 << 20, dtype=torch.uint8, device=dev)
        dst = torch.empty_like(src)
        capi.fill(src, 256 << 20, capi.DT_INT8, capi.FILL_INT8_UNIFORM, 1.0, 1, sptr)
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    # ---------------- headline: bf16 4096^3, A row-major, B column-major, f32 out ----------------
    M = N = K = 4096
    flops = 2.0 * M * N * K
    r = timed(capi.BF16BF16F32, M, N, K, capi.ROW_MAJOR, capi.COL_MAJOR, args.steps, args.warmup)
    plan = capi.plan(capi.BF16BF16F32, M, N, K, capi.ROW_MAJOR, capi.COL_MAJOR).as_dict()
    value = flops / (r["wall_ms"] * 1e-3) / 1e12
    achieved = flops / (r["kernel_ms_mean"] * 1e-3) / 1e12

    out = {
        "metric": "TFLOPS/TOPS at bf16 4096^3 and s8 8192^3; % of MFMA peak; GB/s skinny M",
        "value": round(value, 2),
        "unit": "TFLOPS (bf16 4096^3)",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(r["wall_ms"], 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": "bf16 x bf16 -> f32 GEMM M=N=K=4096, A row-major, B column-major, N(0,1) inputs, "
                               "alpha=1 beta=0, fp32 accumulate",
                   "rotating_input_sets": r["sets"], "plan": plan,
                   "settle": f"{SETTLE_SECONDS} s of back-to-back launches ({r['settle_launches']}) after the warm-up, "
                             "independent of --warmup",
                   "timed_region": f"{r['timed_blocks']} blocks of {args.steps} launches back to back "
                                   f"(>= {MIN_TIMED_SECONDS} s); ms_per_step is their mean",
                   "kernel_ms": "HIP events on the launch stream before and after each timed block, summed over the blocks "
                                "and divided by the launches (the same launches as ms_per_step)"},
        "roofline": {"bound": "mfma", "achieved": round(achieved, 2), "peak": PEAK_TFLOPS["bf16"], "unit": "TFLOP/s",
                     "frac": round(achieved / PEAK_TFLOPS["bf16"], 4), "traffic": measured_traffic(),
                     "traffic_source": "not measured in this run: profiles/mfma_bf16_4096_traffic.json, rocprofv3 --pmc "
                                       "FETCH_SIZE x 2.000 + WRITE_SIZE x 1.000 (KiB per dispatch, scaled by a plain copy)",
                     "kernel_ms_mean": round(r["kernel_ms_mean"], 5),
                     "single_launch_event_pair_ms_mean": round(r["single_launch_ms_mean"], 5),
                     "single_launch_event_pair_ms_median": round(r["single_launch_ms_median"], 5)},
    }

    # ---------------- side measurements named by the metric ----------------
    if not args.no_extras:
        extras = {}
        m8 = 8192
        r8 = timed(capi.S8S8S32, m8, m8, m8, capi.ROW_MAJOR, capi.COL_MAJOR, 30, 40)
        tops = 2.0 * m8 ** 3 / (r8["kernel_ms_mean"] * 1e-3) / 1e12
        extras["s8_8192"] = {"tops": round(tops, 2), "frac_of_int8_peak": round(tops / PEAK_TFLOPS["s8"], 4),
                             "kernel_ms_mean": round(r8["kernel_ms_mean"], 5)}
        # the reference's own bench setting (alpha = beta = 1, C read as well) and its layout (row-major B)
        rb = timed(capi.BF16BF16F32, M, N, K, capi.ROW_MAJOR, capi.COL_MAJOR, args.steps, args.warmup, beta=1)
        extras["bf16_4096_alpha1_beta1"] = {"tflops": round(flops / (rb["kernel_ms_mean"] * 1e-3) / 1e12, 2),
                                            "kernel_ms_mean": round(rb["kernel_ms_mean"], 5)}
        rr = timed(capi.BF16BF16F32, M, N, K, capi.ROW_MAJOR, capi.ROW_MAJOR, args.steps, args.warmup)
        extras["bf16_4096_row_row"] = {"tflops": round(flops / (rr["kernel_ms_mean"] * 1e-3) / 1e12, 2),
                                       "kernel_ms_mean": round(rr["kernel_ms_mean"], 5)}
        # column-major A with column-major B: the same kernel on the transposed problem
        rc = timed(capi.BF16BF16F32, M, N, K, capi.COL_MAJOR, capi.COL_MAJOR, args.steps, args.warmup)
        extras["bf16_4096_col_col"] = {"tflops": round(flops / (rc["kernel_ms_mean"] * 1e-3) / 1e12, 2),
                                       "kernel_ms_mean": round(rc["kernel_ms_mean"], 5)}
        # next row of the scope: fp8 e4m3 x e4m3 -> fp16 (the reference times cuBLASLt on it,
        # nvidia/bench/bench_cublaslt_e4m3.cu:6-21), this library's own kernel on the reference drivers' layout
        # (row-major A and B); inputs N(0, 0.25) so that the fp16 outputs of K = 8192 stay far from overflow
        rf = timed(capi.E4M3E4M3F16, m8, m8, m8, capi.ROW_MAJOR, capi.ROW_MAJOR, 30, 40, scale_b=0.25)
        tf8 = 2.0 * m8 ** 3 / (rf["kernel_ms_mean"] * 1e-3) / 1e12
        extras["e4m3_8192_row_row"] = {"tflops": round(tf8, 2), "frac_of_fp8_peak": round(tf8 / PEAK_TFLOPS["fp8"], 4),
                                       "kernel_ms_mean": round(rf["kernel_ms_mean"], 5)}
        # the type of the reference's own ladder drivers: fp32 4096^3, row-major A and B, full-precision MFMA
        r32 = timed(capi.F32F32F32, M, N, K, capi.ROW_MAJOR, capi.ROW_MAJOR, 20, 20)
        t32 = flops / (r32["kernel_ms_mean"] * 1e-3) / 1e12
        extras["f32_4096_row_row"] = {"tflops": round(t32, 2), "frac_of_f32_peak": round(t32 / PEAK_TFLOPS["f32"], 4),
                                      "kernel_ms_mean": round(r32["kernel_ms_mean"], 5)}
        # the small cubes of the same drivers (nvidia/bench/bench_tiling.cu and its siblings start at 128^3): 64 x 64
        # tiles, so that a grid of a few dozen output tiles still reaches every compute unit
        small = {}
        for sz in (512, 1024, 2048):
            rsm = timed(capi.F32F32F32, sz, sz, sz, capi.ROW_MAJOR, capi.ROW_MAJOR, 100, 100)
            small[str(sz)] = {"tflops": round(2.0 * sz ** 3 / (rsm["kernel_ms_mean"] * 1e-3) / 1e12, 2),
                              "kernel_us_mean": round(rsm["kernel_ms_mean"] * 1e3, 2)}
        extras["f32_small_cubes_row_row"] = small
        # the two remaining configurations of the baseline: int8 1024^3 (row-major A and B) and the ragged fp16
        # problem 4095 x 4097 x 1023 (row-major A and B, predicated edge tiles, unaligned rows)
        rs1 = timed(capi.S8S8S32, 1024, 1024, 1024, capi.ROW_MAJOR, capi.ROW_MAJOR, 100, 100)
        extras["s8_1024_row_row"] = {"tops": round(2.0 * 1024 ** 3 / (rs1["kernel_ms_mean"] * 1e-3) / 1e12, 2),
                                     "kernel_us_mean": round(rs1["kernel_ms_mean"] * 1e3, 2)}
        rg = timed(capi.F16F16F16, 4095, 4097, 1023, capi.ROW_MAJOR, capi.ROW_MAJOR, 50, 50)
        extras["f16_4095x4097x1023_row_row"] = {
            "tflops": round(2.0 * 4095 * 4097 * 1023 / (rg["kernel_ms_mean"] * 1e-3) / 1e12, 2),
            "kernel_us_mean": round(rg["kernel_ms_mean"] * 1e3, 2)}
        # the vendor library beside it (the reference reports cuBLASLt): same operands, same timing, checked the same way
        try:
            functors = importlib.import_module("gemm-zoo_amd.functors")
            lt = functors.HipblasLtGemm(capi.F16F16F16, 4095, 4097, 1023, capi.ROW_MAJOR, capi.ROW_MAJOR)
            rl = timed(capi.F16F16F16, 4095, 4097, 1023, capi.ROW_MAJOR, capi.ROW_MAJOR, 50, 50, vendor=lt)
            extras["hipblaslt_f16_4095x4097x1023_row_row"] = {
                "tflops": round(2.0 * 4095 * 4097 * 1023 / (rl["kernel_ms_mean"] * 1e-3) / 1e12, 2),
                "kernel_us_mean": round(rl["kernel_ms_mean"] * 1e3, 2)}
            lt.close()
            for name, (ty, sz, st, wu, lb, sb) in {
                    "hipblaslt_bf16_4096": (capi.BF16BF16F32, 4096, args.steps, args.warmup, capi.COL_MAJOR, 1.0),
                    "hipblaslt_s8_8192": (capi.S8S8S32, 8192, 30, 40, capi.COL_MAJOR, 1.0),
                    "hipblaslt_e4m3_8192_row_row": (capi.E4M3E4M3F16, 8192, 30, 40, capi.ROW_MAJOR, 0.25),
                    "hipblaslt_f32_4096_row_row": (capi.F32F32F32, 4096, 20, 20, capi.ROW_MAJOR, 1.0)}.items():
                lt = functors.HipblasLtGemm(ty, sz, sz, sz, capi.ROW_MAJOR, lb)
                rl = timed(ty, sz, sz, sz, capi.ROW_MAJOR, lb, st, wu, vendor=lt, scale_b=sb)
                extras[name] = {"tflops": round(2.0 * sz ** 3 / (rl["kernel_ms_mean"] * 1e-3) / 1e12, 2),
                                "kernel_ms_mean": round(rl["kernel_ms_mean"], 5)}
                lt.close()
            small = {}
            for sz in (512, 1024, 2048):
                lt = functors.HipblasLtGemm(capi.F32F32F32, sz, sz, sz, capi.ROW_MAJOR, capi.ROW_MAJOR)
                rl = timed(capi.F32F32F32, sz, sz, sz, capi.ROW_MAJOR, capi.ROW_MAJOR, 100, 100, vendor=lt)
                small[str(sz)] = {"tflops": round(2.0 * sz ** 3 / (rl["kernel_ms_mean"] * 1e-3) / 1e12, 2),
                                  "kernel_us_mean": round(rl["kernel_ms_mean"] * 1e3, 2)}
                lt.close()
            extras["hipblaslt_f32_small_cubes_row_row"] = small
        except Exception as e:  # the comparator is optional: report why it is absent, never fail the bench for it
            extras["hipblaslt"] = {"unavailable": str(e)[:200]}
        sk = {}
        for m in (1, 8, 32, 64, 128):
            rs = timed(capi.BF16BF16BF16, m, 14336, 4096, capi.ROW_MAJOR, capi.COL_MAJOR, 50, 100, scale_b=0.02)
            gbs = rs["problem_bytes"] / (rs["kernel_ms_mean"] * 1e-3) / 1e9
            sk[f"M={m}"] = {"gb_per_s": round(gbs, 1), "frac_of_hbm_peak": round(gbs / PEAK_HBM_GBS, 4),
                            "kernel_us_mean": round(rs["kernel_ms_mean"] * 1e3, 2)}
        extras["skinny_bf16_N14336_K4096"] = sk
        # a long K at 128 rows: the K split with wide column blocks (two launches, partial sums in the workspace)
        rs = timed(capi.BF16BF16BF16, 128, 14336, 14336, capi.ROW_MAJOR, capi.COL_MAJOR, 30, 60, scale_b=0.02)
        gbs = rs["problem_bytes"] / (rs["kernel_ms_mean"] * 1e-3) / 1e9
        extras["skinny_bf16_M128_N14336_K14336"] = {"gb_per_s": round(gbs, 1), "frac_of_hbm_peak": round(gbs / PEAK_HBM_GBS, 4),
                                                    "kernel_us_mean": round(rs["kernel_ms_mean"] * 1e3, 2)}
        out["extras"] = extras

    # ---------------- CPU restatement of the reference GEMM on this box's host cores ----------------
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(M, N, K, args.cpu_seconds)

    print(json.dumps(out))
    return 0


def measured_traffic():
    """HBM bytes per launch of the headline kernel as measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (scaled by a
    plain copy of known size); the figures and the commands that produced them are in profiles/."""
    f = ROOT / "profiles" / "mfma_bf16_4096_traffic.json"
    if not f.exists():
        return None
    try:
        return json.loads(f.read_text())["hbm_bytes_per_launch"]
    except Exception:
        return None


def cpu_baseline(M, N, K, target_seconds):
    """The oracle's literal one-output-per-work-item loop on a band of rows of the same workload."""
    sys.path.insert(0, str(ROOT / "tests"))
    import oracle_lib as O

    threads = int(O.lib.oracle_num_threads())
    a = O.fill(M * K, O.DT_BF16, O.FILL_NORMAL, 1.0, 2025)
    b = O.fill(K * N, O.DT_BF16, O.FILL_NORMAL, 1.0, 2026)
    # calibrate on a few rows, then size the band for about target_seconds
    r0 = max(threads // 4, 2)
    t = time.perf_counter()
    O.gemm(O.BF16BF16F32, a, b, None, M, N, K, O.ROW, O.COL, 1.0, 0.0, threads=threads, rows=(0, r0), naive=True)
    dt = time.perf_counter() - t
    rows = int(min(M, max(r0, target_seconds / max(dt / r0, 1e-9))))
    t = time.perf_counter()
    O.gemm(O.BF16BF16F32, a, b, None, M, N, K, O.ROW, O.COL, 1.0, 0.0, threads=threads, rows=(0, rows), naive=True)
    dt = time.perf_counter() - t
    tflops = 2.0 * rows * N * K / dt / 1e12
    return {"value": round(tflops, 6), "unit": "TFLOPS (bf16 4096^3)", "cores": threads, "kind": "port",
            "sample": f"rows [0,{rows}) of {M} of the same bf16 4096^3 problem ({rows}x{N}x{K} MACs, {dt:.1f} s), "
                      f"literal one-output-per-work-item loop with fp32 accumulate, OpenMP over outputs; "
                      f"full problem would take {dt * M / rows:.0f} s"}


if __name__ == "__main__":
    sys.exit(main())
