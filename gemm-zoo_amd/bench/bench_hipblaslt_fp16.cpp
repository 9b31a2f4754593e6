// Driver of nvidia/bench/bench_cublaslt_fp16.cu:9-24: the vendor library alone (fp16 x fp16 -> fp16, row-major operands).
#include <tuple>

#include "gemm_zoo/benchmark.hpp"

int main() {
  using half_t = gemm_zoo::half_t;
  using kernel_functor_struct = nvidia::kernel_functors::cublasLt_gemm<half_t, half_t>;
  const half_t one{0x3C00};
  benchmark::benchmark<kernel_functor_struct, half_t, half_t>(
      {{128, 128, 128}, {256, 256, 256}, {512, 512, 512}, {1024, 1024, 1024}, {2048, 2048, 2048}, {4096, 4096, 4096},
       {8192, 8192, 8192}},
      one, one);
}
