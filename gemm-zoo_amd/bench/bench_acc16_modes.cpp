// The two opt-in modes that keep the reference kernels' own 16-bit running sum: the shapes of
// nvidia/bench/bench_fp16_mma_gemm.cu:9-27 (fp16 accumulate, nvidia/kernels/sm_80/fp16_mma_gemm.cuh:179) and of
// intel/bench/bench_xe_gemm_bf16_bf16_bf16_m8k16.cpp:10-19 (bf16 accumulate,
// intel/kernels/xe_gemm_bf16_bf16_bf16_m8k16.hpp:88-107), each verified against the any-shape rung in the same mode.
#include <tuple>

#include "gemm_zoo/benchmark.hpp"

int main() {
  using half = gemm_zoo::half_t;
  using half_acc = gemm_zoo::half_acc16_t;
  const half_acc h_one{0x3C00};
  using fp16_kernel = nvidia::kernel_functors::fp16_mma_gemm<half, half_acc, 256, 256, 32>;
  benchmark::benchmark<fp16_kernel, half, half_acc>({{1024, 1024, 1024}, {2048, 2048, 2048}, {4096, 4096, 4096}}, h_one, h_one);

  using bf16_t = gemm_zoo::bf16_t;
  using bf16_acc = gemm_zoo::bf16_acc16_t;
  hipStream_t stream;
  checkHipError(hipStreamCreate(&stream));
  using xe_kernel = intel::gemm_bf16_bf16_bf16_m8k16<bf16_t, bf16_acc>;
  benchmark::benchmark_sizes<xe_kernel, bf16_t, bf16_acc>({{1024, 1024, 1024}, {2048, 2048, 2048}, {4096, 4096, 4096}}, stream);
  checkHipError(hipStreamDestroy(stream));
}
