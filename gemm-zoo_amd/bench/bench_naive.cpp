// Driver of nvidia/bench/bench_naive.cu:9-17 (fp32, sizes 128 ... 1024), then the same for the narrow type bundles.
#include <tuple>

#include "gemm_zoo/benchmark.hpp"

int main() {
  using bf16_t = gemm_zoo::bf16_t;
  std::vector<std::tuple<int, int, int>> sizes = {{128, 128, 128}, {256, 256, 256}, {512, 512, 512}, {1024, 1024, 1024}};
  benchmark::benchmark<nvidia::kernel_functors::naive_gemm<float, float>, float, float>(sizes, 1.0f, 1.0f);
  benchmark::benchmark<nvidia::kernel_functors::naive_gemm<bf16_t, float>, bf16_t, float>(sizes, 1.0f, 1.0f);
  benchmark::benchmark<nvidia::kernel_functors::naive_gemm<int8_t, int32_t>, int8_t, int32_t>(sizes, 1, 1);
}
