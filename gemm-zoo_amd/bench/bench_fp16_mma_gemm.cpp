// Driver of nvidia/bench/bench_fp16_mma_gemm.cu:9-27 (fp16 in and out), plus a ragged shape (4095 x 4097 x 1023).
#include <tuple>

#include "gemm_zoo/benchmark.hpp"

int main() {
  using half = gemm_zoo::half_t;
  constexpr int M = 256, N = 256, K = 32;
  const half one{0x3C00}, zero{0};
  using kernel_functor_struct = nvidia::kernel_functors::fp16_mma_gemm<half, half, M, N, K>;
  benchmark::benchmark<kernel_functor_struct, half, half>(
      {{256, 256, 256}, {512, 512, 512}, {1024, 1024, 1024}, {2048, 2048, 2048}, {4096, 4096, 4096}, {8192, 8192, 8192}},
      one, one);
  benchmark::benchmark<kernel_functor_struct, half, half>({{4095, 4097, 1023}}, one, zero);
}
