// Driver of nvidia/bench/bench_cublaslt_e4m3.cu:6-21: the vendor library alone (fp8 e4m3 x e4m3 -> fp16, row-major operands).
#include <tuple>

#include "gemm_zoo/benchmark.hpp"

int main() {
  using e4m3 = gemm_zoo::e4m3_t;
  using half_t = gemm_zoo::half_t;
  using kernel_functor_struct = nvidia::kernel_functors::cublasLt_gemm<e4m3, half_t>;
  const half_t one{0x3C00};
  benchmark::benchmark<kernel_functor_struct, e4m3, half_t>(
      {{128, 128, 128}, {256, 256, 256}, {512, 512, 512}, {1024, 1024, 1024}, {2048, 2048, 2048}, {4096, 4096, 4096},
       {8192, 8192, 8192}},
      one, one);
}
