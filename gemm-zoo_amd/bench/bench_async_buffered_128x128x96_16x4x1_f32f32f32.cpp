// Driver of nvidia/bench/bench_async_buffered_128x128x96_16x4x1_f32f32f32.cu:9-30 on the functor surface of this build (fp32 x fp32 -> fp32).
#include <tuple>

#include "gemm_zoo/benchmark.hpp"

int main() {
  using kernel_functor_struct = nvidia::kernel_functors::async_buffered_gemm<float, float, 128, 128, 32, 16, 4, 4>;
  benchmark::benchmark<kernel_functor_struct, float, float>(
      {{128, 128, 128}, {256, 256, 256}, {512, 512, 512}, {1024, 1024, 1024}, {2048, 2048, 2048}, {4096, 4096, 4096},
       {8192, 8192, 8192}}, 1.0f, 1.0f);
}
