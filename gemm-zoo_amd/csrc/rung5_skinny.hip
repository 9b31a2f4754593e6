// Rung 5: weight-streaming kernel for decode-shaped problems (M <= 32).
//
// The weight matrix B (N x K, K contiguous) is read exactly once, straight from
// global memory into MFMA operand registers; nothing about it is staged in LDS
// because no element is reused by another wave.  One wavefront owns 16 output
// columns and walks the whole of K in super-steps of 64 elements: the four
// 16-lane groups of the wave each read 32 contiguous bytes of a weight row, so
// every super-step consumes whole 128-byte lines.  Activations (M x K, at most
// 256 KiB) are re-read by every wave and are served by L2.  Loads are issued
// PF super-steps ahead of their use to keep enough bytes in flight to cover
// HBM latency.
//
// v_mfma_f32_16x16x32_{bf16,f16}: the weight fragment is the first operand, so
// a lane ends with 4 consecutive columns of one output row (64-bit stores).
#include "gz_common.hpp"
#include "gz_skinny_cfg.hpp"

namespace gz {

typedef __bf16 sk_bf16x8_t __attribute__((ext_vector_type(8)));
typedef _Float16 sk_f16x8_t __attribute__((ext_vector_type(8)));
typedef float sk_f32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t sk_u32x4_t __attribute__((ext_vector_type(4)));

template <int TYPES>
__device__ inline sk_f32x4_t mfma16(sk_u32x4_t first, sk_u32x4_t second, sk_f32x4_t acc) {
  if constexpr (TYPES == GZ_F16F16F16)
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(sk_f16x8_t, first),
                                                  __builtin_bit_cast(sk_f16x8_t, second), acc, 0, 0, 0);
  else
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(sk_bf16x8_t, first),
                                                   __builtin_bit_cast(sk_bf16x8_t, second), acc, 0, 0, 0);
}

template <int TYPES, int MBLK, int WAVES, int PF>
__global__ void __launch_bounds__(WAVES * 64) skinny_gemm_kernel(GemmArgs<TYPES> g) {
  using T = Traits<TYPES>;
  using in_t = typename T::in_t;
  using out_t = typename T::out_t;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int n_base = (blockIdx.x * WAVES + wave) * SKINNY_COLS_PER_WAVE;
  if (n_base >= g.N) return;  // no barriers in this kernel: a whole wave may leave
  const int r16 = lane & 15, grp = lane >> 4;
  const int K = g.K;

  // Rows past the end are clamped, not zeroed: an output element depends on one
  // row of A and one column of B only, and the clamped ones are never stored.
  const int n_ld = min(n_base + r16, g.N - 1);
  const in_t* __restrict__ bp = g.B + (size_t)n_ld * K + grp * 16;
  const in_t* __restrict__ ap[MBLK];
#pragma unroll
  for (int i = 0; i < MBLK; i++) ap[i] = g.A + (size_t)min(16 * i + r16, g.M - 1) * K + grp * 16;

  sk_f32x4_t acc[MBLK];
#pragma unroll
  for (int i = 0; i < MBLK; i++) acc[i] = sk_f32x4_t{0.f, 0.f, 0.f, 0.f};

  sk_u32x4_t bq[PF][2], aq[PF][MBLK][2];
  const int steps = K / SKINNY_K_STEP;

  auto issue = [&](int slot, int s) {
    const size_t off = (size_t)s * SKINNY_K_STEP;
    bq[slot][0] = __builtin_nontemporal_load(reinterpret_cast<const sk_u32x4_t*>(bp + off));
    bq[slot][1] = __builtin_nontemporal_load(reinterpret_cast<const sk_u32x4_t*>(bp + off + 8));
#pragma unroll
    for (int i = 0; i < MBLK; i++) {
      aq[slot][i][0] = *reinterpret_cast<const sk_u32x4_t*>(ap[i] + off);
      aq[slot][i][1] = *reinterpret_cast<const sk_u32x4_t*>(ap[i] + off + 8);
    }
  };

#pragma unroll
  for (int u = 0; u < PF; u++)
    if (u < steps) issue(u, u);

  for (int s0 = 0; s0 < steps; s0 += PF) {
#pragma unroll
    for (int u = 0; u < PF; u++) {
      const int s = s0 + u;
      if (s < steps) {
        sk_u32x4_t cb[2], ca[MBLK][2];
        cb[0] = bq[u][0];
        cb[1] = bq[u][1];
#pragma unroll
        for (int i = 0; i < MBLK; i++) {
          ca[i][0] = aq[u][i][0];
          ca[i][1] = aq[u][i][1];
        }
        if (s + PF < steps) issue(u, s + PF);
#pragma unroll
        for (int t = 0; t < 2; t++)
#pragma unroll
          for (int i = 0; i < MBLK; i++) acc[i] = mfma16<TYPES>(cb[t], ca[i][t], acc[i]);
      }
    }
  }

  // acc[i][v] = D(16 i + r16, n_base + 4 grp + v)
  const int N = g.N;
  const int n = n_base + 4 * grp;
  const bool vec_ok = (N % 4 == 0) && ((reinterpret_cast<uintptr_t>(g.D) & 15u) == 0) &&
                      (g.beta == 0 || (reinterpret_cast<uintptr_t>(g.C) & 15u) == 0);
#pragma unroll
  for (int i = 0; i < MBLK; i++) {
    const int m = 16 * i + r16;
    if (m >= g.M) continue;
    const size_t o = (size_t)m * N + n;
    if (vec_ok && n + 3 < N) {
      out_t cv[4] = {0, 0, 0, 0}, dv[4];
      if (g.beta != 0) __builtin_memcpy(cv, g.C + o, sizeof(cv));
#pragma unroll
      for (int e = 0; e < 4; e++) dv[e] = epilogue<TYPES>(acc[i][e], g.alpha, g.beta, &cv[e]);
      __builtin_memcpy(g.D + o, dv, sizeof(dv));
    } else {
#pragma unroll
      for (int e = 0; e < 4; e++)
        if (n + e < N) g.D[o + e] = epilogue<TYPES>(acc[i][e], g.alpha, g.beta, g.C + o + e);
    }
  }
}

template <int TYPES> int launch_skinny(const GemmArgs<TYPES>& g, int variant, hipStream_t s) {
  if constexpr (TYPES == GZ_S8S8S32) {
    (void)g; (void)variant; (void)s;
    set_error("skinny rung is built for the 16-bit float types only");
    return GZ_ERR_UNSUPPORTED;
  } else {
    if (variant > 1) {
      set_error("skinny rung has a single variant (got %d)", variant);
      return GZ_ERR_UNSUPPORTED;
    }
    if (!skinny_supported(TYPES, g.M, g.N, g.K, g.layoutA, g.layoutB)) {
      set_error("skinny rung needs row-major A, column-major B, 1 <= M <= %d and K %% %d == 0 (M=%d K=%d)",
                SKINNY_MAX_M, SKINNY_K_STEP, g.M, g.K);
      return GZ_ERR_UNSUPPORTED;
    }
    if ((reinterpret_cast<uintptr_t>(g.A) | reinterpret_cast<uintptr_t>(g.B)) & 15u) {
      set_error("skinny rung needs 16-byte aligned A and B");
      return GZ_ERR_UNSUPPORTED;
    }
    const SkinnyCfg c = skinny_resolve(g.M, g.N, g.K, 256);
    const dim3 grid((unsigned)c.grid_n), block((unsigned)c.threads);
    if (c.mb == 16) hipLaunchKernelGGL((skinny_gemm_kernel<TYPES, 1, 2, 4>), grid, block, 0, s, g);
    else hipLaunchKernelGGL((skinny_gemm_kernel<TYPES, 2, 2, 4>), grid, block, 0, s, g);
    GZ_HIP_TRY(hipGetLastError());
    return GZ_OK;
  }
}

template int launch_skinny<GZ_S8S8S32>(const GemmArgs<GZ_S8S8S32>&, int, hipStream_t);
template int launch_skinny<GZ_BF16BF16F32>(const GemmArgs<GZ_BF16BF16F32>&, int, hipStream_t);
template int launch_skinny<GZ_BF16BF16BF16>(const GemmArgs<GZ_BF16BF16BF16>&, int, hipStream_t);
template int launch_skinny<GZ_F16F16F16>(const GemmArgs<GZ_F16F16F16>&, int, hipStream_t);

}  // namespace gz
