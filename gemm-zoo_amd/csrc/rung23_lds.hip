// Rungs 2 and 3: LDS-tiled GEMM on the vector ALUs.
//
// A work-group of 256 threads owns a 64 x 64 tile of D and walks K in slabs of
// 32.  Both operand slabs sit in LDS widened to the accumulator type and stored
// k-major, As[k][m] and Bs[k][n], with a row pitch of 64 + 4 words: a thread's
// 4 x 4 register block then needs two 128-bit LDS reads per k (a wave reads 16
// distinct B quads = all 64 banks once, and 4 distinct A quads broadcast), and
// the transposing stores of a K-contiguous operand land on distinct banks.
//
// Rung 2 (stages = 1): load slab -> barrier -> compute -> barrier.
// Rung 3 (stages = 2): the global loads of slab t+1 are issued before the math
// of slab t and parked in registers, then written to the other LDS buffer; one
// barrier per slab, memory latency hidden behind the FMAs.
//
// Per output the products are still added in k order: bit-identical to rung 0.
// Stands in for nvidia/kernels/{tiled,rmem_tiled,double_buffered}_gemm.cuh.
#include "gz_common.hpp"

namespace gz {

constexpr int LT_BM = 64, LT_BN = 64, LT_BK = 32, LT_PITCH = 64 + 4, LT_NT = 256;

// One operand slab of 64 lines x 32 k, fetched by 256 threads as 8 elements each.
// KC: lines are K-contiguous (thread -> line tid%64, k-chunk tid/64);
// else: lines run along M/N (thread -> k-line tid/8, 8 consecutive m/n at (tid%8)*8).
template <int TYPES, bool KC> struct SlabLoader {
  using in_t = typename Traits<TYPES>::in_t;
  using acc_t = typename Traits<TYPES>::acc_t;
  in_t r[8];

  // base: matrix; lines_total: M or N; K; ld: elements between its lines; line0: first tile line; k0: first k of slab
  __device__ inline void load(const in_t* __restrict__ base, int lines_total, int K, size_t ld, int line0, int k0, int tid,
                              bool vec_ok) {
    if constexpr (KC) {
      const int line = line0 + (tid & 63), kk = k0 + (tid >> 6) * 8;
      if (line < lines_total && kk + 8 <= K && vec_ok) {
        __builtin_memcpy(r, __builtin_assume_aligned(base + (size_t)line * ld + kk, 8 * sizeof(in_t)), sizeof(r));
      } else {
#pragma unroll
        for (int e = 0; e < 8; e++)
          r[e] = (line < lines_total && kk + e < K) ? base[(size_t)line * ld + kk + e] : (in_t)0;
      }
    } else {
      const int kk = k0 + (tid >> 3), l0 = line0 + (tid & 7) * 8;
      if (kk < K && l0 + 8 <= lines_total && vec_ok) {
        __builtin_memcpy(r, __builtin_assume_aligned(base + (size_t)kk * ld + l0, 8 * sizeof(in_t)),
                         sizeof(r));
      } else {
#pragma unroll
        for (int e = 0; e < 8; e++)
          r[e] = (kk < K && l0 + e < lines_total) ? base[(size_t)kk * ld + l0 + e] : (in_t)0;
      }
    }
  }

  __device__ inline void store(acc_t* lds, int tid) const {
    if constexpr (KC) {
      const int line = tid & 63, kk = (tid >> 6) * 8;
#pragma unroll
      for (int e = 0; e < 8; e++) lds[(kk + e) * LT_PITCH + line] = widen_in<TYPES>(r[e]);
    } else {
      const int kk = tid >> 3, l0 = (tid & 7) * 8;
#pragma unroll
      for (int e = 0; e < 8; e++) lds[kk * LT_PITCH + l0 + e] = widen_in<TYPES>(r[e]);
    }
  }
};

template <int TYPES, bool A_KC, bool B_KC, int STAGES>
// second launch bound: at least 4 waves per SIMD, i.e. at most 128 VGPRs -- without it the double-buffered
// instantiation hoists every LDS read of a slab above the FMAs and ends up with one wave per SIMD
__global__ void __launch_bounds__(LT_NT, 4) lds_gemm_kernel(GemmArgs<TYPES> g) {
  using T = Traits<TYPES>;
  using in_t = typename T::in_t;
  using acc_t = typename T::acc_t;
  typedef acc_t acc4_t __attribute__((ext_vector_type(4)));
  constexpr int SLAB = LT_BK * LT_PITCH;  // words per operand slab
  __shared__ __attribute__((aligned(16))) acc_t lds[STAGES * 2 * SLAB];

  const int tid = threadIdx.x;
  const int tx = tid & 15, ty = tid >> 4;
  const int m0 = blockIdx.y * LT_BM, n0 = blockIdx.x * LT_BN;
  const int M = g.M, N = g.N, K = g.K;

  // vector global loads need 8-element lines starting on their natural alignment
  constexpr uintptr_t VB = 8 * sizeof(in_t) - 1;
  const size_t lda = (size_t)g.lda, ldb = (size_t)g.ldb;
  const bool a_vec = ((A_KC ? K : M) % 8 == 0) && (lda % 8 == 0) && ((reinterpret_cast<uintptr_t>(g.A) & VB) == 0);
  const bool b_vec = ((B_KC ? K : N) % 8 == 0) && (ldb % 8 == 0) && ((reinterpret_cast<uintptr_t>(g.B) & VB) == 0);

  SlabLoader<TYPES, A_KC> la;
  SlabLoader<TYPES, B_KC> lb;

  RunningSum<TYPES> sum[4][4];

  const int slabs = (K + LT_BK - 1) / LT_BK;

  auto compute = [&](const acc_t* as, const acc_t* bs, int k_left) {   // k_left: K minus the slab's first k
#pragma unroll 8
    for (int k = 0; k < LT_BK; k++) {
      const acc4_t a = *reinterpret_cast<const acc4_t*>(as + k * LT_PITCH + ty * 4);
      const acc4_t b = *reinterpret_cast<const acc4_t*>(bs + k * LT_PITCH + tx * 4);
#pragma unroll
      for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 4; j++) {
          sum[i][j].mac(a[i], b[j], k, k_left);  // slabs are whole chunks of the 16-bit running sums
        }
    }
  };

  if constexpr (STAGES == 1) {
    for (int t = 0; t < slabs; t++) {
      la.load(g.A, M, K, lda, m0, t * LT_BK, tid, a_vec);
      lb.load(g.B, N, K, ldb, n0, t * LT_BK, tid, b_vec);
      la.store(lds, tid);
      lb.store(lds + SLAB, tid);
      __syncthreads();
      compute(lds, lds + SLAB, K - t * LT_BK);
      __syncthreads();
    }
  } else {
    if (slabs > 0) {
      la.load(g.A, M, K, lda, m0, 0, tid, a_vec);
      lb.load(g.B, N, K, ldb, n0, 0, tid, b_vec);
      la.store(lds, tid);
      lb.store(lds + SLAB, tid);
    }
    __syncthreads();
    for (int t = 0; t < slabs; t++) {
      acc_t* cur = lds + (t & 1) * 2 * SLAB;
      acc_t* nxt = lds + ((t + 1) & 1) * 2 * SLAB;
      const bool more = t + 1 < slabs;
      if (more) {  // global loads in flight while the FMAs below run
        la.load(g.A, M, K, lda, m0, (t + 1) * LT_BK, tid, a_vec);
        lb.load(g.B, N, K, ldb, n0, (t + 1) * LT_BK, tid, b_vec);
      }
      compute(cur, cur + SLAB, K - t * LT_BK);
      if (more) {
        la.store(nxt, tid);
        lb.store(nxt + SLAB, tid);
      }
      __syncthreads();
    }
  }

#pragma unroll
  for (int i = 0; i < 4; i++) {
    const int m = m0 + ty * 4 + i;
    if (m >= M) continue;
#pragma unroll
    for (int j = 0; j < 4; j++) {
      const int n = n0 + tx * 4 + j;
      if (n < N) {
        g.D[(size_t)m * g.ldd + n] = epilogue<TYPES>(sum[i][j].finish(0), g.alpha, g.beta, g.C + (size_t)m * g.ldc + n);
      }
    }
  }
}

template <int TYPES, int STAGES> static int launch_lds(const GemmArgs<TYPES>& g, int variant, hipStream_t s) {
  if (variant != 0) {
    set_error("LDS rungs have a single variant (got %d)", variant);
    return GZ_ERR_UNSUPPORTED;
  }
  const dim3 block(LT_NT), grid(ceil_div(g.N, LT_BN), ceil_div(g.M, LT_BM));
  if (grid.y > 65535u) {
    set_error("LDS rung: M=%d needs more than 65535 block rows", g.M);
    return GZ_ERR_UNSUPPORTED;
  }
  const bool akc = g.layoutA == GZ_ROW_MAJOR, bkc = g.layoutB == GZ_COL_MAJOR;
  if (akc && bkc) hipLaunchKernelGGL((lds_gemm_kernel<TYPES, true, true, STAGES>), grid, block, 0, s, g);
  else if (akc && !bkc) hipLaunchKernelGGL((lds_gemm_kernel<TYPES, true, false, STAGES>), grid, block, 0, s, g);
  else if (!akc && bkc) hipLaunchKernelGGL((lds_gemm_kernel<TYPES, false, true, STAGES>), grid, block, 0, s, g);
  else hipLaunchKernelGGL((lds_gemm_kernel<TYPES, false, false, STAGES>), grid, block, 0, s, g);
  GZ_HIP_TRY(hipGetLastError());
  return GZ_OK;
}

template <int TYPES> int launch_lds_tiled(const GemmArgs<TYPES>& g, int variant, hipStream_t s) {
  return launch_lds<TYPES, 1>(g, variant, s);
}
template <int TYPES> int launch_double_buffered(const GemmArgs<TYPES>& g, int variant, hipStream_t s) {
  return launch_lds<TYPES, 2>(g, variant, s);
}

#define GZ_INST(TY)                                                                       \
  template int launch_lds_tiled<TY>(const GemmArgs<TY>&, int, hipStream_t);               \
  template int launch_double_buffered<TY>(const GemmArgs<TY>&, int, hipStream_t);
GZ_INST(GZ_S8S8S32)
GZ_INST(GZ_BF16BF16F32)
GZ_INST(GZ_BF16BF16BF16)
GZ_INST(GZ_F16F16F16)
GZ_INST(GZ_F32F32F32)
GZ_INST(GZ_E4M3E4M3F16)
GZ_INST(GZ_E5M2E5M2F16)
GZ_INST(GZ_BF16BF16BF16_ACC16)
GZ_INST(GZ_F16F16F16_ACC16)
#undef GZ_INST

}  // namespace gz
