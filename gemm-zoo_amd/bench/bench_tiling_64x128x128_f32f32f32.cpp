// Driver of nvidia/bench/bench_tiling_64x128x128_f32f32f32.cu:9-20 on the functor surface of this build (fp32 x fp32 -> fp32).
#include <tuple>

#include "gemm_zoo/benchmark.hpp"

int main() {
  using kernel_functor_struct = nvidia::kernel_functors::smem_tiled_gemm<float, float, 64, 128, 128>;
  benchmark::benchmark<kernel_functor_struct, float, float>({{1024, 1024, 1024}, {2048, 2048, 2048}, {4096, 4096, 4096}}, 1.0f, 1.0f);
}
