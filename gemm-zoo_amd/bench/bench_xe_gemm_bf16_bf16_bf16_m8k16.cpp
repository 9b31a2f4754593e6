// Driver of intel/bench/bench_xe_gemm_bf16_bf16_bf16_m8k16.cpp:10-19, plus the decode shapes
// (weights column-major, reported in GB/s).
#include <tuple>

#include "gemm_zoo/benchmark.hpp"

int main() {
  hipStream_t stream;
  checkHipError(hipStreamCreate(&stream));
  using bf16_t = gemm_zoo::bf16_t;
  using kernel = intel::gemm_bf16_bf16_bf16_m8k16<bf16_t, bf16_t>;
  benchmark::benchmark_sizes<kernel, bf16_t, bf16_t>({{1024, 1024, 1024}, {2048, 2048, 2048}, {4096, 4096, 4096}}, stream);
  constexpr auto row = gemm_zoo::layout::row_major, col = gemm_zoo::layout::col_major;
  using decode = intel::gemm_bf16_bf16_bf16_m8k16<bf16_t, bf16_t, row, col>;
  const bf16_t one{0x3F80}, zero{0};
  benchmark::benchmark<decode, bf16_t, bf16_t, row, col>({{1, 14336, 4096}, {8, 14336, 4096}, {32, 14336, 4096}, {128, 14336, 4096}},
                                                        one, zero);
  checkHipError(hipStreamDestroy(stream));
}
