// fp8 x fp8 -> fp16 on this library's own matrix-core kernels, on the sizes of nvidia/bench/bench_cublaslt_e4m3.cu:13-19
// (the reference has no kernel of its own for these types): e4m3 first, then e5m2, row-major operands, alpha = beta = 1.
#include <tuple>

#include "gemm_zoo/benchmark.hpp"

template <typename TIn> static void run() {
  using half_t = gemm_zoo::half_t;
  using kernel_functor_struct = nvidia::kernel_functors::fp8_mma_gemm<TIn, half_t>;
  const half_t one{0x3C00};
  benchmark::benchmark<kernel_functor_struct, TIn, half_t>(
      {{256, 256, 256}, {512, 512, 512}, {1024, 1024, 1024}, {2048, 2048, 2048}, {4096, 4096, 4096}, {8192, 8192, 8192}},
      one, one);
}

int main() {
  run<gemm_zoo::e4m3_t>();
  run<gemm_zoo::e5m2_t>();
}
