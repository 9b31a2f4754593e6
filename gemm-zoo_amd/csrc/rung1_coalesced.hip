// Rung 1: layout-aware lane mapping and wide global loads, still no LDS.
//
// A work-group of 256 threads owns a 16 x 64 tile of D; the 64 lanes of a wave
// lie along N and every thread carries 4 rows.  K is walked in vectors of 16
// bytes:
//   * an operand whose lines are K-contiguous (row-major A, column-major B) is
//     fetched with one 128-bit load per lane and line;
//   * an operand whose lines run along M or N is fetched element by element with
//     the lanes along the contiguous direction, so a wave reads whole lines
//     (B row-major) or one broadcast address (A column-major).
// Each output still sums its products in k order, so the result is bit-identical
// to rung 0.
#include "gz_common.hpp"

namespace gz {

template <int TYPES, bool A_KC, bool B_KC>
__global__ void __launch_bounds__(256) coalesced_gemm_kernel(GemmArgs<TYPES> g) {
  using T = Traits<TYPES>;
  using in_t = typename T::in_t;
  using acc_t = typename T::acc_t;
  constexpr int EPV = 16 / (int)sizeof(in_t);
  constexpr int TM = 4;
  const int M = g.M, N = g.N, K = g.K;
  const int n = blockIdx.x * 64 + (threadIdx.x & 63);
  const int m0 = blockIdx.y * 16 + (threadIdx.x >> 6) * TM;
  const int n_ld = min(n, N - 1);  // clamped lanes compute a value nobody stores

  RunningSum<TYPES> sum[TM];

  // 128-bit loads need every line start on a 16-byte boundary
  const size_t lda = (size_t)g.lda, ldb = (size_t)g.ldb;
  const bool a_vec = A_KC && (K % EPV == 0) && (lda % EPV == 0) && ((reinterpret_cast<uintptr_t>(g.A) & 15u) == 0);
  const bool b_vec = B_KC && (K % EPV == 0) && (ldb % EPV == 0) && ((reinterpret_cast<uintptr_t>(g.B) & 15u) == 0);

  for (int k0 = 0; k0 < K; k0 += EPV) {
    in_t av[TM][EPV], bv[EPV];
    const int kn = min(EPV, K - k0);
    // ---- A ----
#pragma unroll
    for (int r = 0; r < TM; r++) {
      const int m = min(m0 + r, M - 1);
      if constexpr (A_KC) {
        const in_t* p = g.A + (size_t)m * lda + k0;
        if (a_vec) {
          __builtin_memcpy(av[r], __builtin_assume_aligned(p, 16), 16);
        } else {
#pragma unroll
          for (int e = 0; e < EPV; e++) av[r][e] = e < kn ? p[e] : (in_t)0;
        }
      } else {
#pragma unroll
        for (int e = 0; e < EPV; e++) av[r][e] = e < kn ? g.A[(size_t)(k0 + e) * lda + m] : (in_t)0;
      }
    }
    // ---- B ----
    if constexpr (B_KC) {
      const in_t* p = g.B + (size_t)n_ld * ldb + k0;
      if (b_vec) {
        __builtin_memcpy(bv, __builtin_assume_aligned(p, 16), 16);
      } else {
#pragma unroll
        for (int e = 0; e < EPV; e++) bv[e] = e < kn ? p[e] : (in_t)0;
      }
    } else {
#pragma unroll
      for (int e = 0; e < EPV; e++) bv[e] = e < kn ? g.B[(size_t)(k0 + e) * ldb + n_ld] : (in_t)0;
    }
    // ---- multiply-accumulate in k order (zero-filled tail elements add exact zeros) ----
#pragma unroll
    for (int e = 0; e < EPV; e++) {
      const acc_t b = widen_in<TYPES>(bv[e]);
#pragma unroll
      for (int r = 0; r < TM; r++) {
        const acc_t a = widen_in<TYPES>(av[r][e]);
        sum[r].mac(a, b, k0 + e, K);
      }
    }
  }

  if (n < N) {
#pragma unroll
    for (int r = 0; r < TM; r++) {
      const int m = m0 + r;
      if (m < M) {
        g.D[(size_t)m * g.ldd + n] = epilogue<TYPES>(sum[r].finish((K + EPV - 1) / EPV * EPV), g.alpha, g.beta, g.C + (size_t)m * g.ldc + n);
      }
    }
  }
}

template <int TYPES> int launch_coalesced(const GemmArgs<TYPES>& g, int variant, hipStream_t s) {
  if (variant != 0) {
    set_error("coalesced rung has a single variant (got %d)", variant);
    return GZ_ERR_UNSUPPORTED;
  }
  const dim3 block(256), grid(ceil_div(g.N, 64), ceil_div(g.M, 16));
  if (grid.y > 65535u) {
    set_error("coalesced rung: M=%d needs more than 65535 block rows", g.M);
    return GZ_ERR_UNSUPPORTED;
  }
  const bool akc = g.layoutA == GZ_ROW_MAJOR, bkc = g.layoutB == GZ_COL_MAJOR;
  if (akc && bkc) hipLaunchKernelGGL((coalesced_gemm_kernel<TYPES, true, true>), grid, block, 0, s, g);
  else if (akc && !bkc) hipLaunchKernelGGL((coalesced_gemm_kernel<TYPES, true, false>), grid, block, 0, s, g);
  else if (!akc && bkc) hipLaunchKernelGGL((coalesced_gemm_kernel<TYPES, false, true>), grid, block, 0, s, g);
  else hipLaunchKernelGGL((coalesced_gemm_kernel<TYPES, false, false>), grid, block, 0, s, g);
  GZ_HIP_TRY(hipGetLastError());
  return GZ_OK;
}

template int launch_coalesced<GZ_S8S8S32>(const GemmArgs<GZ_S8S8S32>&, int, hipStream_t);
template int launch_coalesced<GZ_BF16BF16F32>(const GemmArgs<GZ_BF16BF16F32>&, int, hipStream_t);
template int launch_coalesced<GZ_BF16BF16BF16>(const GemmArgs<GZ_BF16BF16BF16>&, int, hipStream_t);
template int launch_coalesced<GZ_F16F16F16>(const GemmArgs<GZ_F16F16F16>&, int, hipStream_t);
template int launch_coalesced<GZ_F32F32F32>(const GemmArgs<GZ_F32F32F32>&, int, hipStream_t);
template int launch_coalesced<GZ_E4M3E4M3F16>(const GemmArgs<GZ_E4M3E4M3F16>&, int, hipStream_t);
template int launch_coalesced<GZ_E5M2E5M2F16>(const GemmArgs<GZ_E5M2E5M2F16>&, int, hipStream_t);
template int launch_coalesced<GZ_BF16BF16BF16_ACC16>(const GemmArgs<GZ_BF16BF16BF16_ACC16>&, int, hipStream_t);
template int launch_coalesced<GZ_F16F16F16_ACC16>(const GemmArgs<GZ_F16F16F16_ACC16>&, int, hipStream_t);

}  // namespace gz
