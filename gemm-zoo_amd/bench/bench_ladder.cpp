// Every rung of the ladder on one shape per type bundle (the reference has one driver per rung:
// nvidia/bench/bench_{naive,tiling_*,rmem_*,double_buffered_*,async_buffered_*,bf16_mma_gemm}.cu).
#include <tuple>

#include "gemm_zoo/benchmark.hpp"

template <typename TIn, typename TOut> void ladder(const char* name, int size, TOut one, TOut zero) {
  namespace kf = gemm_zoo::kernel_functors;
  constexpr auto row = gemm_zoo::layout::row_major, col = gemm_zoo::layout::col_major;
  std::vector<std::tuple<int, int, int>> s = {{size, size, size}};
  printf("== %s, A row-major, B column-major ==\n", name);
  printf("naive           "); benchmark::benchmark<kf::naive_gemm<TIn, TOut, row, col>, TIn, TOut, row, col>(s, one, zero, 5);
  printf("coalesced       "); benchmark::benchmark<kf::coalesced_gemm<TIn, TOut, row, col>, TIn, TOut, row, col>(s, one, zero, 5);
  printf("lds_tiled       "); benchmark::benchmark<kf::smem_tiled_gemm<TIn, TOut, 64, 64, 32, row, col>, TIn, TOut, row, col>(s, one, zero, 10);
  printf("double_buffered "); benchmark::benchmark<kf::double_buffered_gemm<TIn, TOut, 64, 64, 32, 4, 4, 1, row, col>, TIn, TOut, row, col>(s, one, zero, 10);
  printf("mfma            "); benchmark::benchmark<kf::auto_gemm<TIn, TOut, row, col>, TIn, TOut, row, col>(s, one, zero, 20);
  printf("hipBLASLt       "); benchmark::benchmark<kf::hipblasLt_gemm<TIn, TOut, row, col>, TIn, TOut, row, col>(s, one, zero, 20);
}

int main() {
  ladder<gemm_zoo::bf16_t, float>("bf16 x bf16 -> f32", 2048, 1.0f, 0.0f);
  ladder<int8_t, int32_t>("s8 x s8 -> s32", 2048, 1, 0);
  ladder<gemm_zoo::half_t, gemm_zoo::half_t>("fp16 x fp16 -> fp16", 2048, gemm_zoo::half_t{0x3C00}, gemm_zoo::half_t{0});
}
