// Driver of nvidia/bench/bench_tf32_mma_gemm.cu:9-26 on the functor surface of this build (fp32 x fp32 -> fp32).
#include <tuple>

#include "gemm_zoo/benchmark.hpp"

int main() {
  using kernel_functor_struct = nvidia::kernel_functors::tf32_mma_gemm<float, float, 128, 128, 32>;
  benchmark::benchmark<kernel_functor_struct, float, float>(
      {{128, 128, 128}, {256, 256, 256}, {512, 512, 512}, {1024, 1024, 1024}, {2048, 2048, 2048}, {4096, 4096, 4096},
       {8192, 8192, 8192}}, 1.0f, 1.0f);
}
