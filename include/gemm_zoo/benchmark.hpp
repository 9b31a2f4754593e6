// gemm-zoo's benchmark / verify harness on HIP.
//
// benchmark::benchmark<Kernel, TIn, TOut>(sizes, alpha, beta, reps) keeps the shape of
// nvidia/utils/benchmark.cuh:111-126 (one stream per run, per-size benchmark_impl :17-108) and
// benchmark::benchmark_sizes<Kernel, TIn, TOut>(sizes, stream, reps) that of intel/bench/benchmark.hpp:117-128
// (alpha = beta = 1).  Per problem size:
//   * P = floor(256 MB / problem bytes) + 1 rotating (A, B, C) sets, so that the Infinity Cache cannot serve
//     the operands (the reference sizes this on l2CacheSize, nvidia/utils/benchmark.cuh:27-38);
//   * seeded device fill, seeds 2025, 2026, ... (intel/bench/benchmark.hpp:66-71);
//   * run once and verify: first against hipBLASLt, on any failure of that against the any-shape fallback
//     kernel (nvidia/utils/benchmark.cuh:56-71); a mismatch throws std::runtime_error("verification failed");
//   * max(reps, P) timed launches, one hipEvent pair each (:73-88);
//   * one line per problem in the reference's format (:97-98) extended with TFLOPS on 2mnk, GB/s and the
//     medians.
#pragma once

#include <hip/hip_runtime_api.h>

#include <algorithm>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <stdexcept>
#include <tuple>
#include <vector>

#include "kernel_functors.hpp"

// nvidia/defines.hpp:6-14
#define checkHipError(call)                                                                          \
  do {                                                                                               \
    hipError_t err_ = (call);                                                                        \
    if (err_ != hipSuccess) {                                                                        \
      printf("HIP error at %s:%d: %s\n", __FILE__, __LINE__, hipGetErrorString(err_));               \
      exit(EXIT_FAILURE);                                                                            \
    }                                                                                                \
  } while (0)

namespace benchmark {

constexpr std::size_t kInfinityCacheBytes = 256u * 1000u * 1000u;

namespace detail {

template <typename T> struct elem;  // gz_fill / gz_compare element codes
template <> struct elem<int8_t> { static constexpr int dt = 0, kind = 0; };
template <> struct elem<gemm_zoo::bf16_t> { static constexpr int dt = 1, kind = 1; };
template <> struct elem<gemm_zoo::half_t> { static constexpr int dt = 2, kind = 1; };
template <> struct elem<gemm_zoo::bf16_acc16_t> { static constexpr int dt = 1, kind = 1; };
template <> struct elem<gemm_zoo::half_acc16_t> { static constexpr int dt = 2, kind = 1; };
template <> struct elem<float> { static constexpr int dt = 3, kind = 1; };
template <> struct elem<int32_t> { static constexpr int dt = 4, kind = 0; };
template <> struct elem<gemm_zoo::e4m3_t> { static constexpr int dt = 5, kind = 1; };
template <> struct elem<gemm_zoo::e5m2_t> { static constexpr int dt = 6, kind = 1; };

struct result {
  double mean_ms, median_ms, gflops_ref, tflops, gbps;
};

template <class Kernel, typename TIn, typename TOut, gemm_zoo::layout LA = gemm_zoo::layout::row_major,
          gemm_zoo::layout LB = gemm_zoo::layout::row_major>
result benchmark_impl(std::size_t m, std::size_t n, std::size_t k, TOut alpha, TOut beta, hipStream_t stream,
                      const int num_repititions, bool verify = true) {
  const int device_id = 0;
  hipDeviceProp_t properties;
  hipError_t err = hipGetDeviceProperties(&properties, device_id);
  if (err != hipSuccess) throw std::runtime_error(hipGetErrorString(err));

  const std::size_t problem_size = m * k * sizeof(TIn) + k * n * sizeof(TIn) + m * n * sizeof(TOut);
  const std::size_t num_problems_required = kInfinityCacheBytes / problem_size + 1;
  const std::size_t min_repitions_required =
      std::max(static_cast<std::size_t>(num_repititions), num_problems_required);

  std::vector<TIn*> a_matrices(num_problems_required, nullptr), b_matrices(num_problems_required, nullptr);
  std::vector<TOut*> c_matrices(num_problems_required, nullptr);
  TOut *d_out = nullptr, *d_ref = nullptr;
  uint64_t seed = 2025;
  for (std::size_t i = 0; i < num_problems_required; i++) {
    checkHipError(hipMalloc(&a_matrices[i], m * k * sizeof(TIn)));
    checkHipError(hipMalloc(&b_matrices[i], n * k * sizeof(TIn)));
    checkHipError(hipMalloc(&c_matrices[i], m * n * sizeof(TOut)));
    gz_fill(a_matrices[i], (int64_t)(m * k), elem<TIn>::dt, elem<TIn>::kind, 1.0f, seed++, stream);
    gz_fill(b_matrices[i], (int64_t)(k * n), elem<TIn>::dt, elem<TIn>::kind, 1.0f, seed++, stream);
    gz_fill(c_matrices[i], (int64_t)(m * n), elem<TOut>::dt, elem<TOut>::kind, 1.0f, seed++, stream);
  }
  checkHipError(hipMalloc(&d_out, m * n * sizeof(TOut)));
  checkHipError(hipMalloc(&d_ref, m * n * sizeof(TOut)));

  Kernel kernel(m, n, k, properties);
  kernel(a_matrices[0], b_matrices[0], c_matrices[0], d_out, alpha, beta, stream);
  checkHipError(hipGetLastError());
  checkHipError(hipStreamSynchronize(stream));
  if (verify) {
    try {
      gemm_zoo::kernel_functors::hipblasLt_gemm<TIn, TOut, LA, LB> reference_gemm(m, n, k, properties);
      reference_gemm(a_matrices[0], b_matrices[0], c_matrices[0], d_ref, alpha, beta, stream);
    } catch (...) {
      gemm_zoo::kernel_functors::generic_gemm<TIn, TOut, LA, LB> reference_gemm(m, n, k);
      reference_gemm(a_matrices[0], b_matrices[0], c_matrices[0], d_ref, alpha, beta, stream);
    }
    checkHipError(hipStreamSynchronize(stream));
    // integers must agree exactly (intel/test/utils.hpp:57); fp32 outputs within the reference's absolute 0.5
    // (nvidia/utils/compare.cuh:19); 16-bit outputs, whose rounding step grows with the value, within 1e-2
    // relative plus 1e-2 of the output scale -- the parity tests hold the kernels to the real tolerances
    float threshold = 0.5f, relative = 0.0f;
    if constexpr (std::is_same_v<TOut, int32_t>) threshold = 0.0f;
    else if constexpr (sizeof(TOut) == 2) { threshold = 1e-2f * std::sqrt((float)k); relative = 1e-2f; }
    // 16-bit running sums: two summation orders part ways wherever a chunk sum's last fp32 bits move a rounding of
    // the running sum, by one spacing of the 16-bit type at the size the sum has then (about sqrt(k), up to 4-5
    // times that in 2^24 outputs); a few such events per output are allowed
    if constexpr (std::is_same_v<TOut, gemm_zoo::half_acc16_t>) threshold = 8.0f * 0x1p-11f * 5.0f * std::sqrt((float)k);
    if constexpr (std::is_same_v<TOut, gemm_zoo::bf16_acc16_t>) threshold = 8.0f * 0x1p-8f * 5.0f * std::sqrt((float)k);
    int64_t different = 0;
    const int st = gz_compare_rel(d_out, d_ref, (int64_t)(m * n), elem<TOut>::dt, threshold, relative, &different,
                                  stream);
    if (st != GZ_OK) throw std::runtime_error(std::string("verification failed: ") + gz_last_error());
  }

  hipEvent_t start, stop;
  checkHipError(hipEventCreate(&start));
  checkHipError(hipEventCreate(&stop));
  std::vector<float> times;
  float total_time = 0;
  for (std::size_t i = 0; i < min_repitions_required; i++) {
    float t = 0;
    const std::size_t pointer_to_use = (i + 1) % a_matrices.size();
    checkHipError(hipEventRecord(start, stream));
    kernel(a_matrices[pointer_to_use], b_matrices[pointer_to_use], c_matrices[pointer_to_use], d_out, alpha, beta,
           stream);
    checkHipError(hipEventRecord(stop, stream));
    checkHipError(hipEventSynchronize(stop));
    checkHipError(hipEventElapsedTime(&t, start, stop));
    total_time += t;
    times.push_back(t);
  }
  std::sort(times.begin(), times.end());
  result r;
  r.mean_ms = total_time / min_repitions_required;
  r.median_ms = times[times.size() / 2];
  const double flops_ref = static_cast<double>(m) * n * (2.0 * k + 3.0);  // the reference's convention
  r.gflops_ref = flops_ref * 1e-9 / (r.mean_ms * 1e-3);
  r.tflops = 2.0 * m * n * k * 1e-12 / (r.mean_ms * 1e-3);
  r.gbps = static_cast<double>(problem_size) * 1e-9 / (r.mean_ms * 1e-3);
  printf("GEMM Problem: [m: %lu n: %lu k: %lu], GFLOPS: %f  Time in ms: %f | 2mnk TFLOPS: %.2f  GB/s: %.1f  "
         "median ms: %f  sets: %lu\n",
         m, n, k, r.gflops_ref, r.mean_ms, r.tflops, r.gbps, r.median_ms, num_problems_required);

  checkHipError(hipEventDestroy(start));
  checkHipError(hipEventDestroy(stop));
  (void)hipFree(d_out);
  (void)hipFree(d_ref);
  for (std::size_t i = 0; i < a_matrices.size(); i++) {
    (void)hipFree(a_matrices[i]);
    (void)hipFree(b_matrices[i]);
    (void)hipFree(c_matrices[i]);
  }
  return r;
}
}  // namespace detail

template <class Kernel, typename TIn, typename TOut, gemm_zoo::layout LA = gemm_zoo::layout::row_major,
          gemm_zoo::layout LB = gemm_zoo::layout::row_major>
void benchmark(std::vector<std::tuple<int, int, int>> problem_sizes, TOut alpha, TOut beta,
               const int num_repititions = 50) {
  hipStream_t stream;
  hipError_t err = hipStreamCreate(&stream);
  if (err != hipSuccess) throw std::runtime_error("Failed to create HIP stream:");
  for (const auto& size_tuple : problem_sizes) {
    auto [m, n, k] = size_tuple;
    detail::benchmark_impl<Kernel, TIn, TOut, LA, LB>(m, n, k, alpha, beta, stream, num_repititions);
  }
  (void)hipStreamDestroy(stream);
}

template <class Kernel, typename TIn, typename TOut, gemm_zoo::layout LA = gemm_zoo::layout::row_major,
          gemm_zoo::layout LB = gemm_zoo::layout::row_major>
void benchmark_sizes(const std::vector<std::tuple<std::size_t, std::size_t, std::size_t>>& sizes, hipStream_t stream,
                     const int num_repititions = 50) {
  TOut alpha, beta;
  if constexpr (std::is_same_v<TOut, gemm_zoo::bf16_t> || std::is_same_v<TOut, gemm_zoo::bf16_acc16_t>) { alpha.bits = beta.bits = 0x3F80; }
  else if constexpr (std::is_same_v<TOut, gemm_zoo::half_t> || std::is_same_v<TOut, gemm_zoo::half_acc16_t>) { alpha.bits = beta.bits = 0x3C00; }
  else { alpha = beta = static_cast<TOut>(1); }
  for (const auto& [m, n, k] : sizes)
    detail::benchmark_impl<Kernel, TIn, TOut, LA, LB>(m, n, k, alpha, beta, stream, num_repititions);
}

}  // namespace benchmark
