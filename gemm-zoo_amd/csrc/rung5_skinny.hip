// Rung 5: weight-streaming kernels for decode-shaped problems (M <= 128).
//
// The weight matrix B (N x K, K contiguous) is read exactly once and nothing about it is reused by another
// wave, so the kernel is a streaming read of B with a little matrix-core work attached.  What decides its
// speed on MI355X (measured):
//   * a compute unit sustains only a limited number of outstanding memory requests, so the chip's bandwidth is
//     reached only when every compute unit streams its equal share: the columns are dealt out in equal
//     groups of at most 32, 4-column granular, one or two groups per compute unit (cols_per_wg);
//   * rows of B are a multiple of 4 KiB apart for the usual K, so work-groups that walk K in step all hit the
//     same L2 / memory channel at the same moment: every work-group starts at a different K chunk (rot);
//   * each byte is used once: the copies carry the non-temporal hint.
//
// skinny_dtl_kernel (M <= 16, K % 128 == 0): a work-group of KS waves owns up to 32 columns; its waves take the
// 128-element K chunks round-robin.  A wave moves its chunk of the 32 rows (8 KiB) from global memory straight
// into a private LDS ring with global_load_lds_dwordx4 -- every instruction moves four 256-byte row pieces --
// and reads the MFMA fragments back with ds_read_b128; the 16-byte pieces of a row are XOR-swizzled with the
// row number on the way in, so the reads are bank-conflict free.  There is no barrier in the main loop and
// S stages are in flight per wave; the waits are hand-counted (the compiler does not see LDS-DMA).  The K
// partial sums of the KS waves meet in LDS at the end.  Activations (at most 16 rows) come from L2 into
// registers with the same depth.
//
// skinny_reg_kernel (M <= 16, K % 64 == 0 only): the earlier design, B straight into MFMA operand registers.
//
// stream_wide_kernel + stream_wide_reduce_kernel (64 < M <= 128, K >= 8192): stream_tile_kernel with column blocks of
// up to 256 columns and K split in two or four parts, so that a compute unit pulls a part of A instead of all of it;
// the parts meet in a workspace and a second launch adds them in a fixed order (gz_skinny_cfg.hpp says when).
//
// stream_tile_kernel (16 < M <= 128, K % 64 == 0): here the activations no longer fit a wave's registers and every
// compute unit needs all of them, so they are shared through LDS.  One work-group per compute unit owns up to 64
// columns.  Four producer waves move stage after stage (64 K elements: A rows and B rows, 128 bytes each, swizzled)
// into a ring with direct-to-LDS copies; four consumer waves read the fragments and run v_mfma_f32_32x32x16.
// Splitting the roles matters: a copy instruction occupies its wave for about 55 cycles however many lanes it
// moves, and with one wave per SIMD doing both jobs the copy issue, the LDS reads and the MFMAs of a stage ran
// back to back.  One barrier per stage says both "stage i has landed" and "stage i - 1 may be overwritten".
//
// v_mfma_f32_16x16x32_{bf16,f16}: the weight fragment is the first operand, so a lane ends with 4 consecutive
// columns of one output row (64-bit stores).
#include "gz_common.hpp"
#include <type_traits>
#include <utility>

#include "gz_skinny_cfg.hpp"

namespace gz {

typedef __bf16 sk_bf16x8_t __attribute__((ext_vector_type(8)));
typedef _Float16 sk_f16x8_t __attribute__((ext_vector_type(8)));
typedef float sk_f32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t sk_u32x4_t __attribute__((ext_vector_type(4)));
typedef float sk_f32x16_t __attribute__((ext_vector_type(16)));

template <int TYPES>
__device__ inline sk_f32x4_t mfma16(sk_u32x4_t first, sk_u32x4_t second, sk_f32x4_t acc) {
  if constexpr (TYPES == GZ_F16F16F16)
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(sk_f16x8_t, first),
                                                  __builtin_bit_cast(sk_f16x8_t, second), acc, 0, 0, 0);
  else
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(sk_bf16x8_t, first),
                                                   __builtin_bit_cast(sk_bf16x8_t, second), acc, 0, 0, 0);
}

template <int TYPES>
__device__ inline sk_f32x16_t mfma32x16(sk_u32x4_t first, sk_u32x4_t second, sk_f32x16_t acc) {
  if constexpr (TYPES == GZ_F16F16F16)
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(sk_f16x8_t, first),
                                                  __builtin_bit_cast(sk_f16x8_t, second), acc, 0, 0, 0);
  else
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(sk_bf16x8_t, first),
                                                   __builtin_bit_cast(sk_bf16x8_t, second), acc, 0, 0, 0);
}

template <int TYPES, int MBLK, int WAVES, int PF>
__global__ void __launch_bounds__(WAVES * 64) skinny_reg_kernel(GemmArgs<TYPES> g) {
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
  const in_t* __restrict__ bp = g.B + (size_t)n_ld * (size_t)g.ldb + grp * 16;
  const in_t* __restrict__ ap[MBLK];
#pragma unroll
  for (int i = 0; i < MBLK; i++) ap[i] = g.A + (size_t)min(16 * i + r16, g.M - 1) * (size_t)g.lda + grp * 16;

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
  const bool vec_ok = (g.ldd % 4 == 0) && (g.beta == 0 || g.ldc % 4 == 0) && ((reinterpret_cast<uintptr_t>(g.D) & 15u) == 0) &&
                      (g.beta == 0 || (reinterpret_cast<uintptr_t>(g.C) & 15u) == 0);
#pragma unroll
  for (int i = 0; i < MBLK; i++) {
    const int m = 16 * i + r16;
    if (m >= g.M) continue;
    const size_t o = (size_t)m * (size_t)g.ldd + n, oc = (size_t)m * (size_t)g.ldc + n;
    if (vec_ok && n + 3 < N) {
      out_t cv[4] = {0, 0, 0, 0}, dv[4];
      if (g.beta != 0) __builtin_memcpy(cv, g.C + oc, sizeof(cv));
#pragma unroll
      for (int e = 0; e < 4; e++) dv[e] = epilogue<TYPES>(acc[i][e], g.alpha, g.beta, &cv[e]);
      __builtin_memcpy(g.D + o, dv, sizeof(dv));
    } else {
#pragma unroll
      for (int e = 0; e < 4; e++)
        if (n + e < N) g.D[o + e] = epilogue<TYPES>(acc[i][e], g.alpha, g.beta, g.C + oc + e);
    }
  }
}


// ---------------------------------------------------------------------------------------------------------
// Direct-to-LDS streaming kernel
// ---------------------------------------------------------------------------------------------------------
template <class F, int... I> __device__ __forceinline__ void sk_for_impl(F&& f, std::integer_sequence<int, I...>) {
  (f(std::integral_constant<int, I>{}), ...);
}
template <int N, class F> __device__ __forceinline__ void sk_for(F&& f) {
  sk_for_impl(f, std::make_integer_sequence<int, N>{});
}
template <int OFF> __device__ __forceinline__ void sk_ds_read16(sk_u32x4_t& dst, uint32_t addr) {
  asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "i"(OFF));
}
__device__ __forceinline__ void sk_set_m0(uint32_t lds_addr) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0" : : "s"(lds_addr) : "memory");
}
// 64 lanes x 16 bytes, global (sbase + voff + OFF) -> LDS (M0 + OFF + 16 * lane); lanes outside `mask` move nothing
// but the instruction still takes its place in the vmcnt order
template <int OFF> __device__ __forceinline__ void sk_copy16(uint32_t voff, const void* sbase_minus_off, uint64_t mask) {
  static_assert(OFF >= -4096 && OFF <= 4095, "13-bit signed immediate");
  asm volatile("s_mov_b64 exec, %3\n\tglobal_load_lds_dwordx4 %0, %1 offset:%2 nt\n\ts_mov_b64 exec, -1"
               :
               : "v"(voff), "s"(sbase_minus_off), "i"(OFF), "s"(mask)
               : "memory");
}
// the same without the non-temporal hint (activations are re-read by every compute unit: keep them in L2)
template <int OFF>
__device__ __forceinline__ void sk_copy16_keep(uint32_t voff, const void* sbase_minus_off, uint64_t mask) {
  static_assert(OFF >= -4096 && OFF <= 4095, "13-bit signed immediate");
  asm volatile("s_mov_b64 exec, %3\n\tglobal_load_lds_dwordx4 %0, %1 offset:%2\n\ts_mov_b64 exec, -1"
               :
               : "v"(voff), "s"(sbase_minus_off), "i"(OFF), "s"(mask)
               : "memory");
}
template <int OFF> __device__ __forceinline__ void sk_load16(sk_u32x4_t& dst, uint32_t voff, const void* sbase) {
  asm volatile("global_load_dwordx4 %0, %1, %2 offset:%3" : "=&v"(dst) : "v"(voff), "s"(sbase), "i"(OFF) : "memory");
}
template <int N> __device__ __forceinline__ void sk_wait_vm() { asm volatile("s_waitcnt vmcnt(%0)" : : "i"(N) : "memory"); }
__device__ __forceinline__ void sk_wait_lgkm0() { asm volatile("s_waitcnt lgkmcnt(0)" : : : "memory"); }
template <int N> __device__ __forceinline__ void sk_wait_lgkm() {
  static_assert(N >= 0 && N <= 15, "lgkmcnt is a 4-bit counter");
  asm volatile("s_waitcnt lgkmcnt(%0)" : : "i"(N) : "memory");
}
// orders later uses of a register after the asm statements that precede this one
__device__ __forceinline__ void sk_touch(sk_u32x4_t& v) { asm volatile("" : "+v"(v)); }

template <int TYPES, int MBLK, int KS, int S>
__global__ void __launch_bounds__(KS * 64) skinny_dtl_kernel(GemmArgs<TYPES> g, int cols_per_wg) {
  using T = Traits<TYPES>;
  using out_t = typename T::out_t;
  extern __shared__ __attribute__((aligned(1024))) char sk_lds[];
  constexpr int CB = 2;                          // 16-column MFMA blocks per work-group
  constexpr int NCP = CB * 4;                    // 1 KiB copies per stage (4 rows x 256 bytes each)
  constexpr int STAGE = SKINNY_DTL_STAGE_BYTES;  // 32 rows x 256 bytes
  constexpr int PER = NCP + 4 * MBLK;            // vector-memory instructions per stage
  constexpr int NA = MBLK * CB;
  static_assert((S - 1) * PER < 64, "vmcnt is a 6-bit counter");
  const uint32_t lds_base = (uint32_t)(uintptr_t)sk_lds;
  const int lane = threadIdx.x & 63;
  const int ks = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int n_base = blockIdx.x * cols_per_wg;
  const int K = g.K, N = g.N, M = g.M;
  const uint32_t ring = lds_base + ks * (S * STAGE);
  const size_t rowb = (size_t)g.ldb * 2, rowb_a = (size_t)g.lda * 2;   // bytes between the columns of B and the rows of A

  // copy j moves rows 4j .. 4j+3 of the group: 16 lanes per row; the lane that fills position p of the LDS row
  // fetches piece p ^ (row & 15) of the 256-byte chunk.  The offsets stay below 2^32: a work-group's columns times
  // the pitch of B, the rows of A times its pitch (the launcher checks both).
  uint32_t voff[NCP];
#pragma unroll
  for (int j = 0; j < NCP; j++) {
    const int row = 4 * j + (lane >> 4), p = lane & 15;
    const int n = min(n_base + row, N - 1);
    voff[j] = (uint32_t)((size_t)(n - n_base) * rowb) + (uint32_t)((p ^ (row & 15)) * 16);
  }
  const char* sb = reinterpret_cast<const char*>(g.B) + (size_t)n_base * rowb;
  const int r16 = lane & 15, grp = lane >> 4;
  uint32_t a_voff[MBLK];
#pragma unroll
  for (int mb = 0; mb < MBLK; mb++) a_voff[mb] = (uint32_t)((size_t)min(mb * 16 + r16, M - 1) * rowb_a) + grp * 16;
  const char* sa = reinterpret_cast<const char*>(g.A);
  // fragment of MFMA step t: row r16 of a column block, K piece 4t + grp
  uint32_t b_addr[4];
#pragma unroll
  for (int t = 0; t < 4; t++) b_addr[t] = ring + r16 * 256 + (((t * 4 + grp) ^ r16) * 16);

  sk_f32x4_t acc[MBLK][CB];
#pragma unroll
  for (int mb = 0; mb < MBLK; mb++)
#pragma unroll
    for (int cb = 0; cb < CB; cb++) acc[mb][cb] = sk_f32x4_t{0.f, 0.f, 0.f, 0.f};
  sk_u32x4_t aq[S][MBLK][4];

  const int chunks = K / SKINNY_DTL_K_STEP;
  const int mine = (chunks - ks + KS - 1) / KS;          // this wave's chunks: ks, ks + KS, ... (before rotation)
  const int rot = (int)(blockIdx.x % (unsigned)chunks);

  auto chunk_byte = [&](int i) {
    int c = i * KS + ks + rot;
    if (c >= chunks) c -= chunks;
    return (size_t)c * 256;
  };
  auto issue_copies = [&](auto slot_c, int i) {
    constexpr int SL = decltype(slot_c)::value;
    const size_t kbyte = chunk_byte(i);
    sk_for<CB>([&](auto q_c) {
      constexpr int Q = decltype(q_c)::value;  // four copies share one M0
      sk_set_m0(ring + SL * STAGE + Q * 4096 + 2048);
      sk_for<4>([&](auto j_c) {
        constexpr int J = decltype(j_c)::value;
        // cols_per_wg is a multiple of 4: a copy moves four whole rows or nothing (mask as a scalar register pair)
        const uint32_t on = (uint32_t)__builtin_amdgcn_readfirstlane(4 * (Q * 4 + J) < cols_per_wg ? -1 : 0);
        sk_copy16<(J - 2) * 1024>(voff[Q * 4 + J], sb + kbyte - (J - 2) * 1024, ((uint64_t)on << 32) | on);
      });
    });
  };
  auto issue_a = [&](auto slot_c, int i) {
    constexpr int SL = decltype(slot_c)::value;
    const size_t kbyte = chunk_byte(i);
    sk_for<MBLK>([&](auto mb_c) {
      constexpr int MB = decltype(mb_c)::value;
      sk_for<4>([&](auto t_c) {
        constexpr int TT = decltype(t_c)::value;
        sk_load16<TT * 64>(aq[SL][MB][TT], a_voff[MB], sa + kbyte);
      });
    });
  };

  sk_for<S>([&](auto sl) {
    if (decltype(sl)::value < mine) {
      issue_copies(sl, decltype(sl)::value);
      issue_a(sl, decltype(sl)::value);
    }
  });

  for (int i0 = 0; i0 < mine; i0 += S) {
    sk_for<S>([&](auto sl) {
      constexpr int SL = decltype(sl)::value;
      const int i = i0 + SL;
      if (i < mine) {
        // stage i has landed once at most the S - 1 younger stages are outstanding
        if (i + S - 1 < mine) sk_wait_vm<(S - 1) * PER>();
        else sk_wait_vm<0>();
        sk_u32x4_t bf[CB][4];
        sk_for<CB>([&](auto cb_c) {
          constexpr int CBI = decltype(cb_c)::value;
          sk_for<4>([&](auto t_c) {
            constexpr int TT = decltype(t_c)::value;
            sk_ds_read16<SL * STAGE + CBI * 4096>(bf[CBI][TT], b_addr[TT]);
          });
        });
        sk_wait_lgkm0();
#pragma unroll
        for (int cb = 0; cb < CB; cb++)
#pragma unroll
          for (int t = 0; t < 4; t++) sk_touch(bf[cb][t]);
#pragma unroll
        for (int mb = 0; mb < MBLK; mb++)
#pragma unroll
          for (int t = 0; t < 4; t++) sk_touch(aq[SL][mb][t]);
        const bool more = i + S < mine;
        if (more) issue_copies(sl, i + S);  // the fragments are in registers: the stage buffer is free
#pragma unroll
        for (int t = 0; t < 4; t++)
#pragma unroll
          for (int mb = 0; mb < MBLK; mb++)
#pragma unroll
            for (int cb = 0; cb < CB; cb++) acc[mb][cb] = mfma16<TYPES>(bf[cb][t], aq[SL][mb][t], acc[mb][cb]);
        if (more) issue_a(sl, i + S);
      }
    });
  }

  // every wave has waited for all of its copies (the last stages wait with vmcnt(0)): the rings can be reused
  float* red = reinterpret_cast<float*>(sk_lds);
  if constexpr (KS > 1) {
    __syncthreads();
#pragma unroll
    for (int mb = 0; mb < MBLK; mb++)
#pragma unroll
      for (int cb = 0; cb < CB; cb++)
#pragma unroll
        for (int e = 0; e < 4; e++) red[((ks * NA + mb * CB + cb) * 4 + e) * 64 + lane] = acc[mb][cb][e];
    __syncthreads();
    if (ks != 0) return;
#pragma unroll
    for (int w = 1; w < KS; w++)
#pragma unroll
      for (int mb = 0; mb < MBLK; mb++)
#pragma unroll
        for (int cb = 0; cb < CB; cb++)
#pragma unroll
          for (int e = 0; e < 4; e++) acc[mb][cb][e] += red[((w * NA + mb * CB + cb) * 4 + e) * 64 + lane];
  }

  // acc[mb][cb][v] = D(16 mb + r16, n_base + 16 cb + 4 grp + v)
  const int n_end = min(n_base + cols_per_wg, N);
  const bool vec_ok = (g.ldd % 4 == 0) && (g.beta == 0 || g.ldc % 4 == 0) && ((reinterpret_cast<uintptr_t>(g.D) & 15u) == 0) &&
                      (g.beta == 0 || (reinterpret_cast<uintptr_t>(g.C) & 15u) == 0);
#pragma unroll
  for (int mb = 0; mb < MBLK; mb++) {
    const int m = mb * 16 + r16;
    if (m >= M) continue;
#pragma unroll
    for (int cb = 0; cb < CB; cb++) {
      const int n = n_base + cb * 16 + 4 * grp;
      const size_t o = (size_t)m * (size_t)g.ldd + n, oc = (size_t)m * (size_t)g.ldc + n;
      if (vec_ok && n + 3 < n_end) {
        out_t cv[4] = {0, 0, 0, 0}, dv[4];
        if (g.beta != 0) __builtin_memcpy(cv, g.C + oc, sizeof(cv));
#pragma unroll
        for (int e = 0; e < 4; e++) dv[e] = epilogue<TYPES>(acc[mb][cb][e], g.alpha, g.beta, &cv[e]);
        __builtin_memcpy(g.D + o, dv, sizeof(dv));
      } else {
#pragma unroll
        for (int e = 0; e < 4; e++)
          if (n + e < n_end) g.D[o + e] = epilogue<TYPES>(acc[mb][cb][e], g.alpha, g.beta, g.C + oc + e);
      }
    }
  }
}


// ---------------------------------------------------------------------------------------------------------
// Producer / consumer streaming tile kernel, 16 < M <= 128
//   LDS ring: S stages of [A: 32 MB32 rows | B: 64 rows] x 128 bytes; piece p (16 bytes) of tile row r sits at
//   position p ^ ((r >> 1) & 7), which makes the 32-row fragment reads bank-conflict free.
//   Consumer wave w: column block w & 1; MB32 >= 2: row group w >> 1 (MB32 / 2 blocks of 32 rows), all four
//   k-steps of a stage; MB32 == 1: the wave pairs split the k-steps and add their sums through LDS at the end.
// ---------------------------------------------------------------------------------------------------------
template <int TYPES, int MB32, int S>
__global__ void __launch_bounds__(STREAM_TILE_THREADS) stream_tile_kernel(GemmArgs<TYPES> g, int cols_per_wg) {
  constexpr int NCW = 4;  // consumer waves; the four producer waves follow
  using T = Traits<TYPES>;
  using out_t = typename T::out_t;
  extern __shared__ __attribute__((aligned(1024))) char sk_lds[];
  constexpr int RB = STREAM_TILE_ROW_BYTES, B_BYTES = STREAM_TILE_COLS * RB, A_ROWS = MB32 * 32, A_BYTES = A_ROWS * RB, STAGE = A_BYTES + B_BYTES;
  constexpr int NA = MB32, NB = 2, NCP = NA + NB;      // copies per producer wave and stage
  // NCW consumer waves: 2 column blocks x NRG row groups x KSPLIT shares of the 4 MFMA k-steps of a stage
  constexpr int NRG = MB32 >= 2 ? 2 : 1, NRB = MB32 / NRG, KSPLIT = NCW / (2 * NRG), NT = 4 / KSPLIT;
  static_assert(KSPLIT >= 1 && NT >= 1, "");
  static_assert(MB32 == 1 || MB32 == 2 || MB32 == 4, "");
  static_assert((S - 2) * NCP < 64, "vmcnt");
  const uint32_t lds_base = (uint32_t)(uintptr_t)sk_lds;
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int K = g.K, N = g.N, M = g.M;
  const int n_base = blockIdx.x * cols_per_wg;
  const int n_end = min(n_base + cols_per_wg, N);
  const size_t rowb = (size_t)g.ldb * 2, rowb_a = (size_t)g.lda * 2;   // bytes between the columns of B and the rows of A
  const int nst = K / STREAM_TILE_K_STEP;
  const int rot = (int)(blockIdx.x % (unsigned)nst);

  if (wave >= NCW) {
    // ---------------- producers: wave p moves A rows [8 NA p, 8 NA (p+1)) and B rows [16 p, 16 p + 16) of every stage ----------------
    const int p = wave - NCW;
    uint32_t voffA[NA], voffB[NB];
    uint64_t maskB[NB];
    const int row_in = lane >> 3, pos = lane & 7;
#pragma unroll
    for (int j = 0; j < NA; j++) {
      const int row = (p * NA + j) * 8 + row_in;
      voffA[j] = (uint32_t)((size_t)min(row, M - 1) * rowb_a) + (pos ^ ((row >> 1) & 7)) * 16;
    }
#pragma unroll
    for (int j = 0; j < NB; j++) {
      const int row = (p * NB + j) * 8 + row_in;
      const int n = min(n_base + row, N - 1);
      voffB[j] = (uint32_t)((size_t)(n - n_base) * rowb) + (pos ^ ((row >> 1) & 7)) * 16;
      maskB[j] = __builtin_amdgcn_ballot_w64(n_base + row < n_end);
    }
    const char* sA = reinterpret_cast<const char*>(g.A);
    const char* sB = reinterpret_cast<const char*>(g.B) + (size_t)n_base * rowb;
    int slot = 0;
    auto issue = [&](int s) {   // a stage past the end: every copy masked off but still counted
      const bool exists = s < nst;
      int c = s + rot;
      if (c >= nst) c -= nst;
      if (!exists) c = 0;
      const uint32_t dst = lds_base + (uint32_t)slot * STAGE;
      slot = slot + 1 == S ? 0 : slot + 1;
      sk_set_m0(dst + p * (NA * 1024) + 2048);
      sk_for<NA>([&](auto j_c) {
        constexpr int J = decltype(j_c)::value;
        sk_copy16_keep<(J - 2) * 1024>(voffA[J], sA + (size_t)c * RB - (J - 2) * 1024, __builtin_amdgcn_ballot_w64(exists));
      });
      sk_set_m0(dst + A_BYTES + p * (NB * 1024) + 2048);
      sk_for<NB>([&](auto j_c) {
        constexpr int J = decltype(j_c)::value;
        const uint64_t m = maskB[J] & __builtin_amdgcn_ballot_w64(exists);
        sk_copy16<(J - 2) * 1024>(voffB[J], sB + (size_t)c * RB - (J - 2) * 1024, m);
      });
    };
    for (int s = 0; s < S - 1; s++) issue(s);
    for (int i = 0; i < nst; i++) {
      sk_wait_vm<(S - 2) * NCP>();                 // stage i has landed
      asm volatile("s_barrier" ::: "memory");     // consumers are done with stage i - 1
      issue(i + S - 1);
    }
    sk_wait_vm<0>();
    if constexpr (KSPLIT > 1) { __syncthreads(); __syncthreads(); }
    return;
  }

  // ------------------------------------------- consumers: waves 0..3 -------------------------------------------
  const int r32 = lane & 31, g2 = lane >> 5;
  const int cbw = wave & 1, rb0 = ((wave >> 1) % NRG) * NRB;
  const int kq = (wave >> 1) / NRG, t0 = kq * NT;
  uint32_t b_addr[NT], a_addr[NT];
#pragma unroll
  for (int t = 0; t < NT; t++) {
    const int pp = ((2 * (t + t0) + g2) ^ ((r32 >> 1) & 7)) * 16;
    a_addr[t] = lds_base + (rb0 * 32 + r32) * RB + pp;
    b_addr[t] = lds_base + A_BYTES + (cbw * 32 + r32) * RB + pp;
  }
  sk_f32x16_t acc[NRB];
#pragma unroll
  for (int r = 0; r < NRB; r++)
#pragma unroll
    for (int e = 0; e < 16; e++) acc[r][e] = 0.f;

  uint32_t so = 0;
  for (int i = 0; i < nst; i++) {
    asm volatile("s_barrier" ::: "memory");
    // All fragment reads of the stage are requested at once, k-step by k-step, and the MFMAs of a k-step start as
    // soon as its own fragments are there (LDS reads return in order), instead of one wait for all of them.
    sk_u32x4_t bf[NT], af[NRB][NT];
    sk_for<NT>([&](auto t_c) {
      constexpr int TT = decltype(t_c)::value;
      sk_ds_read16<0>(bf[TT], b_addr[TT] + so);
      sk_for<NRB>([&](auto r_c) {
        constexpr int R = decltype(r_c)::value;
        sk_ds_read16<R * 32 * RB>(af[R][TT], a_addr[TT] + so);
      });
    });
    so = so + STAGE == S * STAGE ? 0 : so + STAGE;
    sk_for<NT>([&](auto t_c) {
      constexpr int TT = decltype(t_c)::value;
      sk_wait_lgkm<(NT - 1 - TT) * (1 + NRB)>();
      sk_touch(bf[TT]);
#pragma unroll
      for (int r = 0; r < NRB; r++) sk_touch(af[r][TT]);
#pragma unroll
      for (int r = 0; r < NRB; r++) acc[r] = mfma32x16<TYPES>(bf[TT], af[r][TT], acc[r]);
    });
  }
  if constexpr (KSPLIT > 1) {
    float* red = reinterpret_cast<float*>(sk_lds);
    __syncthreads();   // every copy has landed and every fragment has been read: the rings are free
    const int tile = wave % (2 * NRG);
    if (kq > 0) {
#pragma unroll
      for (int r = 0; r < NRB; r++)
#pragma unroll
        for (int e = 0; e < 16; e++) red[((((kq - 1) * 2 * NRG + tile) * NRB + r) * 16 + e) * 64 + lane] = acc[r][e];
    }
    __syncthreads();
    if (kq > 0) return;
#pragma unroll
    for (int q = 1; q < KSPLIT; q++)
#pragma unroll
      for (int r = 0; r < NRB; r++)
#pragma unroll
        for (int e = 0; e < 16; e++) acc[r][e] += red[((((q - 1) * 2 * NRG + tile) * NRB + r) * 16 + e) * 64 + lane];
  }

  const bool vec_ok = (g.ldd % 4 == 0) && (g.beta == 0 || g.ldc % 4 == 0) && ((reinterpret_cast<uintptr_t>(g.D) & 15u) == 0) &&
                      (g.beta == 0 || (reinterpret_cast<uintptr_t>(g.C) & 15u) == 0);
#pragma unroll
  for (int r = 0; r < NRB; r++) {
    const int m = (rb0 + r) * 32 + r32;
    if (m >= M) continue;
#pragma unroll
    for (int q = 0; q < 4; q++) {
      const int n = n_base + cbw * 32 + q * 8 + g2 * 4;
      const size_t o = (size_t)m * (size_t)g.ldd + n, oc = (size_t)m * (size_t)g.ldc + n;
      if (vec_ok && n + 3 < n_end) {
        out_t cv[4] = {0, 0, 0, 0}, dv[4];
        if (g.beta != 0) __builtin_memcpy(cv, g.C + oc, sizeof(cv));
#pragma unroll
        for (int e = 0; e < 4; e++) dv[e] = epilogue<TYPES>(acc[r][4 * q + e], g.alpha, g.beta, &cv[e]);
        __builtin_memcpy(g.D + o, dv, sizeof(dv));
      } else {
#pragma unroll
        for (int e = 0; e < 4; e++)
          if (n + e < n_end) g.D[o + e] = epilogue<TYPES>(acc[r][4 * q + e], g.alpha, g.beta, g.C + oc + e);
      }
    }
  }
}

// ---------------------------------------------------------------------------------------------------------
// The producer / consumer kernel with wide column blocks and a split K, 64 < M <= 128 (see skinny_resolve_wide)
//   Work-group b serves K part ks = (b % 8) % KS of column group (b / 8) * (8 / KS) + (b % 8) / KS: work-groups go
//   to the XCDs in turn, so the work-groups of one XCD share a K part of A and its L2 holds that part only.
//   LDS ring: S stages of [A: 128 rows | B: 64 CB rows] x 128 bytes, swizzled as above.  Producer wave p moves A rows
//   [32 p, 32 p + 32) and B rows [16 CB p, 16 CB (p + 1)) of every stage.  Consumer wave w: row blocks 2 (w >> 1) and
//   2 (w >> 1) + 1, the 32-column blocks (w & 1) + 2 c for c < CB, all four k-steps of a stage; the fragments of
//   k-step t + 1 are requested before the MFMAs of k-step t.
//   The sums leave as the waves hold them: slot (ks, group) of the workspace, float4 index
//   (((wave * 2 + r) * CB + c) * 4 + q) * 64 + lane - whole 1 KiB stores; stream_wide_reduce_kernel reads them back in
//   the same order.
// ---------------------------------------------------------------------------------------------------------
template <int TYPES, int CB, int S>
__global__ void __launch_bounds__(STREAM_TILE_THREADS) stream_wide_kernel(GemmArgs<TYPES> g, int cols_per_wg, int groups, int KS,
                                                                          float* ws) {
  constexpr int NCW = 4;
  extern __shared__ __attribute__((aligned(1024))) char sk_lds[];
  constexpr int RB = STREAM_TILE_ROW_BYTES, A_ROWS = 128, A_BYTES = A_ROWS * RB, B_ROWS = STREAM_TILE_COLS * CB;
  constexpr int B_BYTES = B_ROWS * RB, STAGE = A_BYTES + B_BYTES;
  constexpr int NA = 4, NB = 2 * CB, NCP = NA + NB;   // copies per producer wave and stage
  constexpr int NRB = 2, NT = 4;
  static_assert(CB >= 2 && CB <= STREAM_WIDE_MAX_CB, "two to four 64-column blocks");
  static_assert((S - 2) * NCP < 64, "vmcnt");
  static_assert(S * STAGE <= 160 * 1024, "LDS");
  const uint32_t lds_base = (uint32_t)(uintptr_t)sk_lds;
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int N = g.N, M = g.M;
  const int xcd = blockIdx.x % 8;
  const int ks = xcd % KS, cg = ((int)blockIdx.x / 8) * (8 / KS) + xcd / KS;
  if (cg >= groups) return;   // the grid is rounded up to whole rounds of the XCDs; before any barrier
  const int n_base = cg * cols_per_wg;
  const int n_end = min(n_base + cols_per_wg, N);
  const size_t rowb = (size_t)g.ldb * 2, rowb_a = (size_t)g.lda * 2;
  const int nst_all = g.K / STREAM_TILE_K_STEP;
  const int st_q = nst_all / KS, st_r = nst_all % KS;
  const int st0 = ks * st_q + min(ks, st_r), nst = st_q + (ks < st_r ? 1 : 0);
  const int rot = (int)((unsigned)cg % (unsigned)nst);

  if (wave >= NCW) {
    const int p = wave - NCW;
    uint32_t voffA[NA], voffB[NB];
    uint64_t maskB[NB];
    const int row_in = lane >> 3, pos = lane & 7;
#pragma unroll
    for (int j = 0; j < NA; j++) {
      const int row = (p * NA + j) * 8 + row_in;
      voffA[j] = (uint32_t)((size_t)min(row, M - 1) * rowb_a) + (pos ^ ((row >> 1) & 7)) * 16;
    }
#pragma unroll
    for (int j = 0; j < NB; j++) {
      const int row = (p * NB + j) * 8 + row_in;
      const int n = min(n_base + row, N - 1);
      voffB[j] = (uint32_t)((size_t)(n - n_base) * rowb) + (pos ^ ((row >> 1) & 7)) * 16;
      maskB[j] = __builtin_amdgcn_ballot_w64(n_base + row < n_end);
    }
    const char* sA = reinterpret_cast<const char*>(g.A) + (size_t)st0 * RB;
    const char* sB = reinterpret_cast<const char*>(g.B) + (size_t)n_base * rowb + (size_t)st0 * RB;
    int slot = 0;
    auto issue = [&](int s) {   // a stage past the end: every copy masked off but still counted
      const bool exists = s < nst;
      int c = s + rot;
      if (c >= nst) c -= nst;
      if (!exists) c = 0;
      const uint32_t dst = lds_base + (uint32_t)slot * STAGE;
      slot = slot + 1 == S ? 0 : slot + 1;
      sk_set_m0(dst + p * (NA * 1024) + 2048);
      sk_for<NA>([&](auto j_c) {
        constexpr int J = decltype(j_c)::value;
        sk_copy16_keep<(J - 2) * 1024>(voffA[J], sA + (size_t)c * RB - (J - 2) * 1024, __builtin_amdgcn_ballot_w64(exists));
      });
      sk_set_m0(dst + A_BYTES + p * (NB * 1024) + (NB / 2) * 1024);
      sk_for<NB>([&](auto j_c) {
        constexpr int J = decltype(j_c)::value;
        const uint64_t m = maskB[J] & __builtin_amdgcn_ballot_w64(exists);
        sk_copy16<(J - NB / 2) * 1024>(voffB[J], sB + (size_t)c * RB - (J - NB / 2) * 1024, m);
      });
    };
    for (int s = 0; s < S - 1; s++) issue(s);
    for (int i = 0; i < nst; i++) {
      sk_wait_vm<(S - 2) * NCP>();                 // stage i has landed
      asm volatile("s_barrier" ::: "memory");     // consumers are done with stage i - 1
      issue(i + S - 1);
    }
    sk_wait_vm<0>();
    return;
  }

  // consumers
  const int r32 = lane & 31, g2 = lane >> 5;
  const int cbw = wave & 1, rb0 = (wave >> 1) * NRB;
  uint32_t b_addr[NT], a_addr[NT];
#pragma unroll
  for (int t = 0; t < NT; t++) {
    const int pp = ((2 * t + g2) ^ ((r32 >> 1) & 7)) * 16;
    a_addr[t] = lds_base + (rb0 * 32 + r32) * RB + pp;
    b_addr[t] = lds_base + A_BYTES + (cbw * 32 + r32) * RB + pp;
  }
  sk_f32x16_t acc[NRB][CB];
#pragma unroll
  for (int r = 0; r < NRB; r++)
#pragma unroll
    for (int c = 0; c < CB; c++)
#pragma unroll
      for (int e = 0; e < 16; e++) acc[r][c][e] = 0.f;

  uint32_t so = 0;
  for (int i = 0; i < nst; i++) {
    asm volatile("s_barrier" ::: "memory");
    sk_u32x4_t bf[2][CB], af[2][NRB];
    auto request = [&](auto t_c) {
      constexpr int TT = decltype(t_c)::value;
      sk_for<NRB>([&](auto r_c) {
        constexpr int R = decltype(r_c)::value;
        sk_ds_read16<R * 32 * RB>(af[TT & 1][R], a_addr[TT] + so);
      });
      sk_for<CB>([&](auto c_c) {
        constexpr int C = decltype(c_c)::value;
        sk_ds_read16<C * 64 * RB>(bf[TT & 1][C], b_addr[TT] + so);
      });
    };
    request(std::integral_constant<int, 0>{});
    sk_for<NT>([&](auto t_c) {
      constexpr int TT = decltype(t_c)::value;
      if constexpr (TT + 1 < NT) {
        request(std::integral_constant<int, TT + 1>{});
        sk_wait_lgkm<NRB + CB>();
      } else {
        sk_wait_lgkm0();
      }
#pragma unroll
      for (int r = 0; r < NRB; r++) sk_touch(af[TT & 1][r]);
#pragma unroll
      for (int c = 0; c < CB; c++) sk_touch(bf[TT & 1][c]);
#pragma unroll
      for (int r = 0; r < NRB; r++)
#pragma unroll
        for (int c = 0; c < CB; c++) acc[r][c] = mfma32x16<TYPES>(bf[TT & 1][c], af[TT & 1][r], acc[r][c]);
    });
    so = so + STAGE == S * STAGE ? 0 : so + STAGE;
  }

  sk_f32x4_t* out = reinterpret_cast<sk_f32x4_t*>(ws) +
                    ((size_t)ks * groups + cg) * (size_t)(NCW * NRB * CB * 4 * 64) + (size_t)wave * (NRB * CB * 4 * 64) + lane;
#pragma unroll
  for (int r = 0; r < NRB; r++)
#pragma unroll
    for (int c = 0; c < CB; c++)
#pragma unroll
      for (int q = 0; q < 4; q++)
        out[((r * CB + c) * 4 + q) * 64] = sk_f32x4_t{acc[r][c][4 * q], acc[r][c][4 * q + 1], acc[r][c][4 * q + 2], acc[r][c][4 * q + 3]};
}

// Second launch of the split: a work-group per 32 x 32 block of the output.  Its 256 lanes read the block's sums in
// the order the first launch stored them (whole lines), add the K parts in their order, turn the block through LDS
// and write it row by row - eight lanes per row, 128 contiguous bytes of an fp32 D - with alpha, beta and the rounding.
// (One lane per four outputs in storage order, each lane writing its own 16 bytes, took 10 us at M = 128, N = 14336:
// a wave's store then touched 32 rows.)
template <int TYPES>
__global__ void __launch_bounds__(256) stream_wide_reduce_kernel(GemmArgs<TYPES> g, int cols_per_wg, int groups, int KS, int CB,
                                                                 const float* ws) {
  using out_t = typename Traits<TYPES>::out_t;
  __shared__ float tile[32][36];
  const int per_slot = 4 * 2 * CB * 4 * 64;   // float4 per slot
  const int blocks_per_slot = 4 * 2 * CB;
  const int cg = (int)blockIdx.x / blocks_per_slot, blk = (int)blockIdx.x % blocks_per_slot;
  const int c = blk % CB, r = (blk / CB) % 2, wave = blk / (2 * CB);
  const int tid = threadIdx.x, lane = tid % 64, q = tid / 64;
  const sk_f32x4_t* in = reinterpret_cast<const sk_f32x4_t*>(ws) + (size_t)cg * per_slot + (size_t)blk * 256 + tid;
  sk_f32x4_t sum = in[0];
  for (int ks = 1; ks < KS; ks++) {
    const sk_f32x4_t v = in[(size_t)ks * groups * per_slot];
#pragma unroll
    for (int e = 0; e < 4; e++) sum[e] += v[e];
  }
#pragma unroll
  for (int e = 0; e < 4; e++) tile[lane & 31][q * 8 + (lane >> 5) * 4 + e] = sum[e];
  __syncthreads();
  const int row = tid / 8, j = tid % 8;
  const int m = ((wave >> 1) * 2 + r) * 32 + row;
  const int n = cg * cols_per_wg + ((wave & 1) + 2 * c) * 32 + 4 * j;
  const int n_end = min((cg + 1) * cols_per_wg, g.N);
  if (m >= g.M || n >= n_end) return;
  float v[4];
#pragma unroll
  for (int e = 0; e < 4; e++) v[e] = tile[row][4 * j + e];
  const size_t o = (size_t)m * (size_t)g.ldd + n, oc = (size_t)m * (size_t)g.ldc + n;
  const bool vec_ok = (g.ldd % 4 == 0) && (g.beta == 0 || g.ldc % 4 == 0) && ((reinterpret_cast<uintptr_t>(g.D) & 15u) == 0) &&
                      (g.beta == 0 || (reinterpret_cast<uintptr_t>(g.C) & 15u) == 0);
  if (vec_ok && n + 3 < n_end) {
    out_t cv[4] = {0, 0, 0, 0}, dv[4];
    if (g.beta != 0) __builtin_memcpy(cv, g.C + oc, sizeof(cv));
#pragma unroll
    for (int e = 0; e < 4; e++) dv[e] = epilogue<TYPES>(v[e], g.alpha, g.beta, &cv[e]);
    __builtin_memcpy(g.D + o, dv, sizeof(dv));
  } else {
#pragma unroll
    for (int e = 0; e < 4; e++)
      if (n + e < n_end) g.D[o + e] = epilogue<TYPES>(v[e], g.alpha, g.beta, g.C + oc + e);
  }
}

template <int TYPES> int launch_skinny(const GemmArgs<TYPES>& g, int variant, hipStream_t s) {
  if constexpr (TYPES == GZ_S8S8S32 || TYPES == GZ_F32F32F32 || is_fp8(TYPES) || is_acc16(TYPES)) {
    (void)g; (void)variant; (void)s;
    set_error("skinny rung is built for the 16-bit float types with fp32 accumulation only");
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
    if (((reinterpret_cast<uintptr_t>(g.A) | reinterpret_cast<uintptr_t>(g.B)) & 15u) || !skinny_lines_ok(g.lda, g.ldb)) {
      set_error("skinny rung needs 16-byte aligned A and B and leading dimensions that are multiples of 8 elements "
                "(lda=%lld ldb=%lld)", (long long)g.lda, (long long)g.ldb);
      return GZ_ERR_UNSUPPORTED;
    }
    const SkinnyCfg c = skinny_resolve(g.M, g.N, g.K, device_compute_units(), (unsigned long long)workspace_limit());
    const dim3 grid((unsigned)c.grid_n), block((unsigned)c.threads);
    if (c.kind == SKINNY_KIND_TILE_WIDE) {
      void* ws = nullptr;
      const int st = workspace_acquire((size_t)c.workspace_bytes, s, &ws);
      if (st != GZ_OK) return st;
      const int per_round = 8 / c.split_k;   // column groups per round of the eight XCDs
      const dim3 wgrid((unsigned)((c.grid_n + per_round - 1) / per_round * 8));
      auto k2 = stream_wide_kernel<TYPES, 2, STREAM_WIDE_STAGES_2>;
      auto k3 = stream_wide_kernel<TYPES, 3, STREAM_WIDE_STAGES_3>;
      auto k4 = stream_wide_kernel<TYPES, 4, STREAM_WIDE_STAGES_4>;
      auto kern = c.cb == 2 ? k2 : c.cb == 3 ? k3 : k4;
      GZ_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                     c.lds_bytes));
      hipLaunchKernelGGL(kern, wgrid, block, c.lds_bytes, s, g, c.cols_per_wg, c.grid_n, c.split_k, static_cast<float*>(ws));
      GZ_HIP_TRY(hipGetLastError());
      hipLaunchKernelGGL((stream_wide_reduce_kernel<TYPES>), dim3((unsigned)(c.grid_n * 4 * 2 * c.cb)), dim3(256), 0, s, g,
                         c.cols_per_wg, c.grid_n, c.split_k, c.cb, static_cast<const float*>(ws));
    } else if (c.kind == SKINNY_KIND_TILE) {
      auto k1 = stream_tile_kernel<TYPES, 1, STREAM_TILE_STAGES_1>;
      auto k2 = stream_tile_kernel<TYPES, 2, STREAM_TILE_STAGES_2>;
      auto k4 = stream_tile_kernel<TYPES, 4, STREAM_TILE_STAGES_4>;
      auto kern = c.mb == 32 ? k1 : c.mb == 64 ? k2 : k4;
      GZ_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                     c.lds_bytes));
      hipLaunchKernelGGL(kern, grid, block, c.lds_bytes, s, g, c.cols_per_wg);
    } else if (c.kind == SKINNY_KIND_DTL) {
      constexpr int KS = SKINNY_DTL_WAVES, S = SKINNY_DTL_STAGES;
      auto kern = skinny_dtl_kernel<TYPES, 1, KS, S>;
      // more than 64 KiB of dynamic LDS needs the opt-in; harmless below
      GZ_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                     c.lds_bytes));
      hipLaunchKernelGGL(kern, grid, block, c.lds_bytes, s, g, c.cols_per_wg);
    } else {
      hipLaunchKernelGGL((skinny_reg_kernel<TYPES, 1, 2, 4>), grid, block, 0, s, g);
    }
    GZ_HIP_TRY(hipGetLastError());
    return GZ_OK;
  }
}

template int launch_skinny<GZ_S8S8S32>(const GemmArgs<GZ_S8S8S32>&, int, hipStream_t);
template int launch_skinny<GZ_BF16BF16F32>(const GemmArgs<GZ_BF16BF16F32>&, int, hipStream_t);
template int launch_skinny<GZ_BF16BF16BF16>(const GemmArgs<GZ_BF16BF16BF16>&, int, hipStream_t);
template int launch_skinny<GZ_F16F16F16>(const GemmArgs<GZ_F16F16F16>&, int, hipStream_t);
template int launch_skinny<GZ_F32F32F32>(const GemmArgs<GZ_F32F32F32>&, int, hipStream_t);
template int launch_skinny<GZ_E4M3E4M3F16>(const GemmArgs<GZ_E4M3E4M3F16>&, int, hipStream_t);
template int launch_skinny<GZ_E5M2E5M2F16>(const GemmArgs<GZ_E5M2E5M2F16>&, int, hipStream_t);
template int launch_skinny<GZ_BF16BF16BF16_ACC16>(const GemmArgs<GZ_BF16BF16BF16_ACC16>&, int, hipStream_t);
template int launch_skinny<GZ_F16F16F16_ACC16>(const GemmArgs<GZ_F16F16F16_ACC16>&, int, hipStream_t);

}  // namespace gz
