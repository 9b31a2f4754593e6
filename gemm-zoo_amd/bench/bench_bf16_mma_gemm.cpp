// Driver of nvidia/bench/bench_bf16_mma_gemm.cu:9-28 on the gfx950 ladder (same sizes, alpha = beta = 1),
// followed by the headline configuration of this library (B column-major, beta = 0).
#include <tuple>

#include "gemm_zoo/benchmark.hpp"

int main() {
  using bf16_t = gemm_zoo::bf16_t;
  constexpr int M = 128, N = 128, K = 32;
  float alpha = 1.0f, beta = 1.0f;
  using kernel_functor_struct = nvidia::kernel_functors::bf16_mma_gemm<bf16_t, float, M, N, K>;
  benchmark::benchmark<kernel_functor_struct, bf16_t, float>(
      {{256, 256, 256}, {512, 512, 512}, {1024, 1024, 1024}, {2048, 2048, 2048}, {4096, 4096, 4096}, {8192, 8192, 8192}},
      alpha, beta);
  constexpr auto row = gemm_zoo::layout::row_major, col = gemm_zoo::layout::col_major;
  using headline = gemm_zoo::kernel_functors::bf16_mma_gemm<bf16_t, float, 256, 256, 64, row, col>;
  benchmark::benchmark<headline, bf16_t, float, row, col>({{4096, 4096, 4096}, {8192, 8192, 8192}}, 1.0f, 0.0f);
}
