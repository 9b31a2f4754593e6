// Driver of bench/bench_xe_gemm_s8_s8_s32_m8k16.cpp:10-18 (1024^3, 2048^3, 4096^3, alpha = beta = 1), plus the
// 8192^3 shape with column-major B.
#include <tuple>

#include "gemm_zoo/benchmark.hpp"

int main() {
  hipStream_t stream;
  checkHipError(hipStreamCreate(&stream));
  using kernel = intel::gemm_s8_s8_s32_m8k16<int8_t, int32_t>;
  benchmark::benchmark_sizes<kernel, int8_t, int32_t>({{1024, 1024, 1024}, {2048, 2048, 2048}, {4096, 4096, 4096}}, stream);
  constexpr auto row = gemm_zoo::layout::row_major, col = gemm_zoo::layout::col_major;
  using headline = intel::gemm_s8_s8_s32_m8k16<int8_t, int32_t, row, col>;
  benchmark::benchmark<headline, int8_t, int32_t, row, col>({{8192, 8192, 8192}}, 1, 0, 10);
  checkHipError(hipStreamDestroy(stream));
}
