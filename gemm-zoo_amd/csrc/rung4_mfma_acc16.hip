// MFMA rung for the two opt-in modes with a 16-bit running sum (bf16bf16bf16_acc16, f16f16f16_acc16).
//
// The matrix cores of gfx950 accumulate in fp32 only, so the 16-bit accumulator of the reference kernels
// (intel/kernels/xe_gemm_bf16_bf16_bf16_m8k16.hpp:88-97: DPAS with a bf16 C operand, 16 k per instruction;
// nvidia/kernels/sm_80/fp16_mma_gemm.cuh:179: mma.sync.m16n8k8 with an fp16 C operand, 8 k per instruction) is
// rebuilt around them: one MFMA with a zero C operand gives the fp32 sum of one chunk's products
// (v_mfma_f32_32x32x16_bf16 = 16 k, v_mfma_f32_32x32x8_f16 = 8 k), and the vector ALUs fold it into the running sum,
// sum = T(fp32(sum + chunk)), which lives in fp32 registers but always holds a value of the output type.  The fold is
// sixteen adds and roundings per MFMA and lane and takes several times as long as the MFMA itself: the mode is for
// reproducing the reference kernels' numbers, not for speed.
//
// One kernel: 128 x 128 tile, four waves (2 x 2, 64 x 64 each), K slabs of 32 elements.  A slab goes from global
// memory into registers while the previous one is computed, then into one LDS buffer (rows of 64 + 16 bytes).  Any
// layout, any M / N / K and any alignment: loads outside the matrices are zero-filled element by element, chunks
// that start past K are skipped (folding an all-zero chunk would still turn a running sum of -0 into +0).
#include "rung4_mfma.hpp"

namespace gz {

constexpr int A16_BM = 128, A16_BN = 128, A16_BK = 32, A16_PITCH = A16_BK * 2 + 16, A16_THREADS = 256;

typedef _Float16 a16_f16x4_t __attribute__((ext_vector_type(4)));

// Eight consecutive k of one line (row of A / column of B) starting at k0, zero-filled outside the matrix.
// KC: the line is contiguous in memory (row-major A, column-major B); `vec`: 16-byte loads are allowed.
template <bool KC>
__device__ inline u32x4_t a16_fetch8(const uint16_t* __restrict__ base, int line, int lines, int k0, int K, size_t ld, bool vec) {
  u32x4_t v = {0u, 0u, 0u, 0u};
  if (line >= lines || k0 >= K) return v;
  if constexpr (KC) {
    const uint16_t* p = base + (size_t)line * ld + k0;
    if (vec && k0 + 8 <= K) {
      __builtin_memcpy(&v, __builtin_assume_aligned(p, 16), 16);
      return v;
    }
    uint16_t t[8];
#pragma unroll
    for (int e = 0; e < 8; e++) t[e] = k0 + e < K ? p[e] : (uint16_t)0;
    __builtin_memcpy(&v, t, 16);
  } else {
    uint16_t t[8];
#pragma unroll
    for (int e = 0; e < 8; e++) t[e] = k0 + e < K ? base[(size_t)(k0 + e) * ld + line] : (uint16_t)0;
    __builtin_memcpy(&v, t, 16);
  }
  return v;
}

template <int TYPES, bool A_KC, bool B_KC>
__global__ void __launch_bounds__(A16_THREADS) mfma_acc16_kernel(GemmArgs<TYPES> g) {
  using out_t = typename Traits<TYPES>::out_t;
  constexpr bool BF = TYPES == GZ_BF16BF16BF16_ACC16;
  constexpr int CHUNK = acc16_chunk(TYPES), NCHUNK = A16_BK / CHUNK;
  constexpr int FM = 2, FN = 2;
  __shared__ __attribute__((aligned(16))) char lds[(A16_BM + A16_BN) * A16_PITCH];
  char* const lds_a = lds;
  char* const lds_b = lds + A16_BM * A16_PITCH;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int M = g.M, N = g.N, K = g.K;
  const int tiles_n = (N + A16_BN - 1) / A16_BN;
  const int m0 = (int)(blockIdx.x / (unsigned)tiles_n) * A16_BM, n0 = (int)(blockIdx.x % (unsigned)tiles_n) * A16_BN;
  const size_t lda = (size_t)g.lda, ldb = (size_t)g.ldb, ldc = (size_t)g.ldc, ldd = (size_t)g.ldd;
  const bool a_vec = A_KC && (K % 8 == 0) && (lda % 8 == 0) && ((reinterpret_cast<uintptr_t>(g.A) & 15u) == 0);
  const bool b_vec = B_KC && (K % 8 == 0) && (ldb % 8 == 0) && ((reinterpret_cast<uintptr_t>(g.B) & 15u) == 0);

  f32x16_t acc[FM][FN];
#pragma unroll
  for (int i = 0; i < FM; i++)
#pragma unroll
    for (int j = 0; j < FN; j++)
#pragma unroll
      for (int e = 0; e < 16; e++) acc[i][j][e] = 0.f;

  // a slab of one operand is 128 lines x 4 pieces of 8 k: two pieces per thread
  u32x4_t ra[2], rb[2];
  auto fetch = [&](int k0) {
#pragma unroll
    for (int j = 0; j < 2; j++) {
      const int p = tid + A16_THREADS * j, line = p >> 2, q = p & 3;
      ra[j] = a16_fetch8<A_KC>(g.A, m0 + line, M, k0 + 8 * q, K, lda, a_vec);
      rb[j] = a16_fetch8<B_KC>(g.B, n0 + line, N, k0 + 8 * q, K, ldb, b_vec);
    }
  };
  auto park = [&]() {
#pragma unroll
    for (int j = 0; j < 2; j++) {
      const int p = tid + A16_THREADS * j, line = p >> 2, q = p & 3;
      *reinterpret_cast<u32x4_t*>(lds_a + line * A16_PITCH + q * 16) = ra[j];
      *reinterpret_cast<u32x4_t*>(lds_b + line * A16_PITCH + q * 16) = rb[j];
    }
  };

  const int r32 = lane & 31, g2 = lane >> 5;
  const f32x16_t zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  const int slabs = (K + A16_BK - 1) / A16_BK;
  if (slabs > 0) fetch(0);
  for (int t = 0; t < slabs; t++) {
    park();
    __syncthreads();
    if (t + 1 < slabs) fetch((t + 1) * A16_BK);
    const int k_left = K - t * A16_BK;
#pragma unroll
    for (int c = 0; c < NCHUNK; c++) {
      if (c * CHUNK < k_left) {   // the same for every lane of the work-group
        // lane (r32, g2) supplies k = c CHUNK + g2 CHUNK/2 .. + CHUNK/2 of line r32 to both operands
        constexpr int HALF_BYTES = CHUNK;   // CHUNK/2 elements of two bytes
        const int kb = c * CHUNK * 2 + g2 * HALF_BYTES;
        static_for<FM>([&](auto i_c) {
          constexpr int I = decltype(i_c)::value;
          const char* pa = lds_a + (wm * 64 + I * 32 + r32) * A16_PITCH + kb;
          static_for<FN>([&](auto j_c) {
            constexpr int J = decltype(j_c)::value;
            const char* pb = lds_b + (wn * 64 + J * 32 + r32) * A16_PITCH + kb;
            f32x16_t part;
            if constexpr (BF) {
              const bf16x8_t fa = *reinterpret_cast<const bf16x8_t*>(pa);
              const bf16x8_t fb = *reinterpret_cast<const bf16x8_t*>(pb);
              part = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fb, fa, zero, 0, 0, 0);
            } else {
              const a16_f16x4_t fa = *reinterpret_cast<const a16_f16x4_t*>(pa);
              const a16_f16x4_t fb = *reinterpret_cast<const a16_f16x4_t*>(pb);
              part = __builtin_amdgcn_mfma_f32_32x32x8f16(fb, fa, zero, 0, 0, 0);
            }
            static_for<16>([&](auto e_c) {
              constexpr int E = decltype(e_c)::value;
              acc[I][J][E] = round_out<TYPES>(add_rn(acc[I][J][E], part[E]));
            });
          });
        });
      }
    }
    __syncthreads();
  }

  // acc[i][j][4 q + e] = D(m0 + 64 wm + 32 i + r32, n0 + 64 wn + 32 j + 8 q + 4 g2 + e)
  const bool use_c = g.beta != 0;
  const bool vec = (N & 3) == 0 && (ldd & 3) == 0 && (!use_c || (ldc & 3) == 0) &&
                   ((reinterpret_cast<uintptr_t>(g.D) | (use_c ? reinterpret_cast<uintptr_t>(g.C) : 0)) & 7u) == 0;
  static_for<FM>([&](auto i_c) {
    constexpr int I = decltype(i_c)::value;
    const int m = m0 + wm * 64 + I * 32 + r32;
    static_for<FN>([&](auto j_c) {
      constexpr int J = decltype(j_c)::value;
      static_for<4>([&](auto q_c) {
        constexpr int Q = decltype(q_c)::value;
        const int n = n0 + wn * 64 + J * 32 + Q * 8 + g2 * 4;
        if (m >= M || n >= N) return;
        const size_t o = (size_t)m * ldd + n, oc = (size_t)m * ldc + n;
        if (vec) {   // N is a multiple of four: the lane's four columns exist together
          out_t cv[4] = {0, 0, 0, 0}, dv[4];
          if (use_c) __builtin_memcpy(cv, g.C + oc, sizeof(cv));
          dv[0] = epilogue<TYPES>(acc[I][J][4 * Q + 0], g.alpha, g.beta, &cv[0]);
          dv[1] = epilogue<TYPES>(acc[I][J][4 * Q + 1], g.alpha, g.beta, &cv[1]);
          dv[2] = epilogue<TYPES>(acc[I][J][4 * Q + 2], g.alpha, g.beta, &cv[2]);
          dv[3] = epilogue<TYPES>(acc[I][J][4 * Q + 3], g.alpha, g.beta, &cv[3]);
          __builtin_memcpy(g.D + o, dv, sizeof(dv));
        } else {
          if (n + 0 < N) g.D[o + 0] = epilogue<TYPES>(acc[I][J][4 * Q + 0], g.alpha, g.beta, g.C + oc + 0);
          if (n + 1 < N) g.D[o + 1] = epilogue<TYPES>(acc[I][J][4 * Q + 1], g.alpha, g.beta, g.C + oc + 1);
          if (n + 2 < N) g.D[o + 2] = epilogue<TYPES>(acc[I][J][4 * Q + 2], g.alpha, g.beta, g.C + oc + 2);
          if (n + 3 < N) g.D[o + 3] = epilogue<TYPES>(acc[I][J][4 * Q + 3], g.alpha, g.beta, g.C + oc + 3);
        }
      });
    });
  });
}

template <int TYPES> static int launch_acc16(const GemmArgs<TYPES>& g, int variant, hipStream_t s) {
  if (variant > 1) {
    set_error("mfma rung has a single variant for the 16-bit running-sum modes (got %d)", variant);
    return GZ_ERR_UNSUPPORTED;
  }
  const long long tiles = (long long)ceil_div(g.M, A16_BM) * ceil_div(g.N, A16_BN);
  const dim3 grid((unsigned)tiles), block(A16_THREADS);
  const bool a_kc = g.layoutA == GZ_ROW_MAJOR, b_kc = g.layoutB == GZ_COL_MAJOR;
  if (a_kc && b_kc) hipLaunchKernelGGL((mfma_acc16_kernel<TYPES, true, true>), grid, block, 0, s, g);
  else if (a_kc && !b_kc) hipLaunchKernelGGL((mfma_acc16_kernel<TYPES, true, false>), grid, block, 0, s, g);
  else if (!a_kc && b_kc) hipLaunchKernelGGL((mfma_acc16_kernel<TYPES, false, true>), grid, block, 0, s, g);
  else hipLaunchKernelGGL((mfma_acc16_kernel<TYPES, false, false>), grid, block, 0, s, g);
  GZ_HIP_TRY(hipGetLastError());
  return GZ_OK;
}

template <> int launch_mfma<GZ_BF16BF16BF16_ACC16>(const GemmArgs<GZ_BF16BF16BF16_ACC16>& g, int variant, hipStream_t s) {
  return launch_acc16<GZ_BF16BF16BF16_ACC16>(g, variant, s);
}
template <> int launch_mfma<GZ_F16F16F16_ACC16>(const GemmArgs<GZ_F16F16F16_ACC16>& g, int variant, hipStream_t s) {
  return launch_acc16<GZ_F16F16F16_ACC16>(g, variant, s);
}

}  // namespace gz
