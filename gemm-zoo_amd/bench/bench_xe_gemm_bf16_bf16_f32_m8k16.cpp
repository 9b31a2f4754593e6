// Driver of intel/bench/bench_xe_gemm_bf16_bf16_f32_m8k16.cpp:10-19.
#include <tuple>

#include "gemm_zoo/benchmark.hpp"

int main() {
  hipStream_t stream;
  checkHipError(hipStreamCreate(&stream));
  using bf16_t = gemm_zoo::bf16_t;
  using kernel = intel::gemm_bf16_bf16_f32_m8k16<bf16_t, float>;
  benchmark::benchmark_sizes<kernel, bf16_t, float>({{1024, 1024, 1024}, {2048, 2048, 2048}, {4096, 4096, 4096}}, stream);
  checkHipError(hipStreamDestroy(stream));
}
