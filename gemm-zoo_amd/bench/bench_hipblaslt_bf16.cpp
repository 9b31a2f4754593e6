// Driver of nvidia/bench/bench_cublaslt_bf16.cu: the vendor library alone, for the number reported alongside.
#include <tuple>

#include "gemm_zoo/benchmark.hpp"

int main() {
  using bf16_t = gemm_zoo::bf16_t;
  constexpr auto row = gemm_zoo::layout::row_major, col = gemm_zoo::layout::col_major;
  using kernel = nvidia::kernel_functors::cublasLt_gemm<bf16_t, float, row, col>;
  benchmark::benchmark<kernel, bf16_t, float, row, col>({{1024, 1024, 1024}, {2048, 2048, 2048}, {4096, 4096, 4096}, {8192, 8192, 8192}},
                                                       1.0f, 0.0f);
  using kernel8 = nvidia::kernel_functors::cublasLt_gemm<int8_t, int32_t, row, col>;
  benchmark::benchmark<kernel8, int8_t, int32_t, row, col>({{8192, 8192, 8192}}, 1, 0, 10);
}
