"""Host-side mirror of gemm-zoo's benchmark / verify harness (``nvidia/utils/benchmark.cuh:17-126``,
``intel/bench/benchmark.hpp:24-128``): rotating input sets sized against the 256 MB Infinity Cache, seeded device
fill, verify-once against hipBLASLt (fallback: the any-shape LDS rung), one event pair per timed launch, and the
reference's result line.  Device memory and events come from torch; every kernel runs through the C ABI."""
from __future__ import annotations

import math
from dataclasses import dataclass

from . import capi
from .functors import DeviceProps, HipblasLtGemm, KernelFunctor, functor

INFINITY_CACHE_BYTES = 256 * 1000 * 1000


@dataclass
class Result:
    m: int
    n: int
    k: int
    mean_ms: float
    median_ms: float
    gflops_ref: float   # the reference's m*n*(2k+3) convention
    tflops: float       # 2*m*n*k
    gbps: float
    sets: int


def _torch_types(types):
    import torch

    tin = {capi.S8S8S32: torch.int8, capi.BF16BF16F32: torch.bfloat16, capi.BF16BF16BF16: torch.bfloat16,
           capi.F16F16F16: torch.float16, capi.F32F32F32: torch.float32,
           capi.E4M3E4M3F16: torch.float8_e4m3fn, capi.E5M2E5M2F16: torch.float8_e5m2,
           capi.BF16BF16BF16_ACC16: torch.bfloat16, capi.F16F16F16_ACC16: torch.float16}[types]
    tout = {capi.S8S8S32: torch.int32, capi.BF16BF16F32: torch.float32, capi.BF16BF16BF16: torch.bfloat16,
            capi.F16F16F16: torch.float16, capi.F32F32F32: torch.float32,
            capi.E4M3E4M3F16: torch.float16, capi.E5M2E5M2F16: torch.float16,
            capi.BF16BF16BF16_ACC16: torch.bfloat16, capi.F16F16F16_ACC16: torch.float16}[types]
    return tin, tout


_IN_DT = {capi.S8S8S32: capi.DT_INT8, capi.BF16BF16F32: capi.DT_BF16, capi.BF16BF16BF16: capi.DT_BF16,
          capi.F16F16F16: capi.DT_F16, capi.F32F32F32: capi.DT_F32,
          capi.E4M3E4M3F16: capi.DT_E4M3, capi.E5M2E5M2F16: capi.DT_E5M2,
          capi.BF16BF16BF16_ACC16: capi.DT_BF16, capi.F16F16F16_ACC16: capi.DT_F16}
_OUT_DT = {capi.S8S8S32: capi.DT_INT32, capi.BF16BF16F32: capi.DT_F32, capi.BF16BF16BF16: capi.DT_BF16,
           capi.F16F16F16: capi.DT_F16, capi.F32F32F32: capi.DT_F32,
           capi.E4M3E4M3F16: capi.DT_F16, capi.E5M2E5M2F16: capi.DT_F16,
           capi.BF16BF16BF16_ACC16: capi.DT_BF16, capi.F16F16F16_ACC16: capi.DT_F16}


def benchmark_impl(kernel_cls, m, n, k, alpha, beta, stream=None, num_repititions=50, verify=True, quiet=False):
    import torch

    types = kernel_cls.types
    tin, tout = _torch_types(types)
    dev = torch.device("cuda", torch.cuda.current_device())
    stream = stream or torch.cuda.current_stream()
    sptr = stream.cuda_stream
    problem = capi.IN_SIZE[types] * (m * k + k * n) + capi.OUT_SIZE[types] * m * n
    sets = INFINITY_CACHE_BYTES // problem + 1
    reps = max(num_repititions, sets)
    kind_in = capi.FILL_INT8_UNIFORM if types == capi.S8S8S32 else capi.FILL_NORMAL
    seed = 2025
    a_s, b_s, c_s = [], [], []
    for _ in range(sets):
        a = torch.empty(m * k, dtype=tin, device=dev); b = torch.empty(k * n, dtype=tin, device=dev)
        c = torch.empty(m * n, dtype=tout, device=dev)
        capi.fill(a, m * k, _IN_DT[types], kind_in, 1.0, seed, sptr); seed += 1
        capi.fill(b, k * n, _IN_DT[types], kind_in, 1.0, seed, sptr); seed += 1
        capi.fill(c, m * n, _OUT_DT[types], kind_in, 1.0, seed, sptr); seed += 1
        a_s.append(a); b_s.append(b); c_s.append(c)
    d_out = torch.empty(m * n, dtype=tout, device=dev)
    kernel = kernel_cls(m, n, k, DeviceProps.current())
    kernel(a_s[0], b_s[0], c_s[0], d_out, alpha, beta, stream)
    stream.synchronize()
    if verify:
        d_ref = torch.empty_like(d_out)
        try:
            ref = HipblasLtGemm(types, m, n, k, kernel_cls.layout_a, kernel_cls.layout_b)
            ref(a_s[0], b_s[0], c_s[0], d_ref, alpha, beta, stream)
        except Exception:  # like the reference: any failure of the vendor path falls back to the generic kernel
            fb = type("generic", (KernelFunctor,), dict(types=types, layout_a=kernel_cls.layout_a,
                                                        layout_b=kernel_cls.layout_b, rung=capi.RUNG_LDS_TILED))
            fb(m, n, k)(a_s[0], b_s[0], c_s[0], d_ref, alpha, beta, stream)
        if types == capi.S8S8S32:
            thr, rel = 0.0, 0.0
        elif types in (capi.BF16BF16BF16_ACC16, capi.F16F16F16_ACC16):
            # two summation orders of a 16-bit running sum part ways by one spacing of the type (at the size the sum
            # has then, about sqrt(k), up to 4-5 times that among 2^24 outputs) wherever a chunk sum's last fp32
            # bits move a rounding; a few such events per output are allowed
            eps = 2.0 ** -8 if types == capi.BF16BF16BF16_ACC16 else 2.0 ** -11
            thr, rel = 8 * eps * 5 * math.sqrt(k), 1e-2
        elif capi.OUT_SIZE[types] == 2:
            thr, rel = 1e-2 * math.sqrt(k), 1e-2
        else:
            thr, rel = 0.5, 0.0
        if capi.compare(d_out, d_ref, m * n, _OUT_DT[types], thr, sptr, rel):
            raise RuntimeError("verification failed")
    times = []
    for i in range(reps):
        j = (i + 1) % sets
        s = torch.cuda.Event(enable_timing=True); e = torch.cuda.Event(enable_timing=True)
        s.record(stream)
        kernel(a_s[j], b_s[j], c_s[j], d_out, alpha, beta, stream)
        e.record(stream)
        e.synchronize()
        times.append(s.elapsed_time(e))
    mean = sum(times) / len(times)
    med = sorted(times)[len(times) // 2]
    r = Result(m, n, k, mean, med, m * n * (2 * k + 3) * 1e-9 / (mean * 1e-3), 2.0 * m * n * k * 1e-12 / (mean * 1e-3),
               problem * 1e-9 / (mean * 1e-3), sets)
    if not quiet:
        print("GEMM Problem: [m: %d n: %d k: %d], GFLOPS: %f  Time in ms: %f | 2mnk TFLOPS: %.2f  GB/s: %.1f" %
              (m, n, k, r.gflops_ref, r.mean_ms, r.tflops, r.gbps), flush=True)
    return r


def benchmark(kernel_cls, problem_sizes, alpha, beta, num_repititions=50):
    """benchmark::benchmark<Kernel, TIn, TOut>(sizes, alpha, beta, reps) -- nvidia/utils/benchmark.cuh:111-126."""
    import torch

    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        return [benchmark_impl(kernel_cls, m, n, k, alpha, beta, stream, num_repititions) for m, n, k in problem_sizes]


def benchmark_sizes(kernel_cls, sizes, stream=None, num_repititions=50):
    """benchmark::benchmark_sizes<...>(sizes, queue) with alpha = beta = 1 -- intel/bench/benchmark.hpp:117-128."""
    return [benchmark_impl(kernel_cls, m, n, k, 1, 1, stream, num_repititions) for m, n, k in sizes]


__all__ = ["benchmark", "benchmark_sizes", "benchmark_impl", "Result", "functor"]
