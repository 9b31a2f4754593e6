// Driver of nvidia/bench/bench_cublaslt_e5m2.cu:6-21: the vendor library alone (fp8 e5m2 x e5m2 -> fp16, row-major operands).
#include <tuple>

#include "gemm_zoo/benchmark.hpp"

int main() {
  using e5m2 = gemm_zoo::e5m2_t;
  using half_t = gemm_zoo::half_t;
  using kernel_functor_struct = nvidia::kernel_functors::cublasLt_gemm<e5m2, half_t>;
  const half_t one{0x3C00};
  benchmark::benchmark<kernel_functor_struct, e5m2, half_t>(
      {{128, 128, 128}, {256, 256, 256}, {512, 512, 512}, {1024, 1024, 1024}, {2048, 2048, 2048}, {4096, 4096, 4096},
       {8192, 8192, 8192}},
      one, one);
}
