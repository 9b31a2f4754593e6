// Driver of nvidia/bench/bench_cublaslt_tf32.cu:9-24: the vendor library alone on fp32 operands (hipBLASLt computes
// them in full fp32; gfx950 has no tf32 mode).
#include <tuple>

#include "gemm_zoo/benchmark.hpp"

int main() {
  using kernel_functor_struct = nvidia::kernel_functors::cublasLt_gemm<float, float>;
  benchmark::benchmark<kernel_functor_struct, float, float>(
      {{128, 128, 128}, {256, 256, 256}, {512, 512, 512}, {1024, 1024, 1024}, {2048, 2048, 2048}, {4096, 4096, 4096},
       {8192, 8192, 8192}},
      1.0f, 1.0f);
}
