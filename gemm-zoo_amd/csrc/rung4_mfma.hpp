// Rung 4: wavefront-level MFMA GEMM for gfx950.
//
// One work-group owns a BM x BN tile of D and walks K in slabs of 128 bytes per
// row (64 16-bit elements or 128 int8).  Each lane's MFMA operand is 16
// contiguous K-bytes of one row, so a fragment is a single ds_read_b128 whatever
// the element type:
//     v_mfma_f32_32x32x16_{bf16,f16}  (8 elements / lane)
//     v_mfma_i32_32x32x32_i8          (16 elements / lane)
// The B fragment is passed as the instruction's first operand, so every lane
// ends up with 4 consecutive columns of one output row and the epilogue stores
// are 128-bit (fp32 / int32) or 64-bit (16-bit outputs).
//
// The kernels of the rung:
//   mfma_gemm_kernel   general: any layout, any shape (predicated EDGE instantiation), any alignment.
//                      Slabs are staged global -> registers -> LDS ([row][k], pitch 144 B: the 16-byte pad
//                      makes the fragment reads of 16 consecutive rows hit 16 distinct 4-bank groups);
//                      operands whose contiguous dimension is not K (row-major B, column-major A) are
//                      transposed in registers on the way in.  Tiles 256x256, 256x128, 128x128 and, for
//                      grids that those leave mostly empty, 64x64 (16- and 32-bit elements).
//   mfma_dtl_kernel    compiler-scheduled fast path for whole tiles with 16-byte aligned rows: slabs go
//                      global -> LDS directly (global_load_lds_dwordx4), unpadded swizzled rows.
//   mfma_ring16_kernel (rung4_mfma_ring16.hpp) the hand-scheduled kernel with the 16x16 matrix instructions
//                      and a ring of five LDS buffers, on 256 x 256 and 128 x 128 tiles: what the launcher
//                      runs wherever operands are aligned and K is whole slabs.
//
// Stands in for nvidia/kernels/sm_80/{bf16,fp16}_mma_gemm.cuh and
// intel/kernels/xe_gemm_*_m8k16.hpp (same operation, new design).
#pragma once
#include <type_traits>
#include <utility>

#include "gz_common.hpp"
#include "gz_mfma_cfg.hpp"

namespace gz {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef int i32x16_t __attribute__((ext_vector_type(16)));
typedef int i32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));

template <class F, int... I>
__device__ __forceinline__ void static_for_impl(F&& f, std::integer_sequence<int, I...>) {
  (f(std::integral_constant<int, I>{}), ...);
}
template <int N, class F> __device__ __forceinline__ void static_for(F&& f) {
  static_for_impl(f, std::make_integer_sequence<int, N>{});
}

template <int TYPES> struct AccVec { using type = f32x16_t; };
template <> struct AccVec<GZ_S8S8S32> { using type = i32x16_t; };
// accumulators of one 16x16 block
template <int TYPES> struct AccVec4Of { using type = f32x4_t; };
template <> struct AccVec4Of<GZ_S8S8S32> { using type = i32x4_t; };

template <int TYPES>
__device__ inline typename AccVec<TYPES>::type mfma32(u32x4_t first, u32x4_t second,
                                                      typename AccVec<TYPES>::type acc) {
  if constexpr (TYPES == GZ_S8S8S32) {
    return __builtin_amdgcn_mfma_i32_32x32x32_i8(__builtin_bit_cast(i32x4_t, first),
                                                 __builtin_bit_cast(i32x4_t, second), acc, 0, 0, 0);
  } else if constexpr (TYPES == GZ_F16F16F16) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8_t, first),
                                                  __builtin_bit_cast(f16x8_t, second), acc, 0, 0, 0);
  } else if constexpr (is_fp8(TYPES)) {
    // One fragment pair alone (the kernels' own loops for these types pair two K steps instead, see mfma_f8_pair):
    // 16 bytes per lane are 16 K values; v_mfma_f32_32x32x16_{fp8_fp8,bf8_bf8} takes 8 per lane, so the two halves
    // of the fragment pair feed one instruction each (which k a lane's bytes stand for is the same on both
    // operands, and that is all a dot product needs).
    typedef long i64x2_t __attribute__((ext_vector_type(2)));
    const i64x2_t b = __builtin_bit_cast(i64x2_t, first), a = __builtin_bit_cast(i64x2_t, second);
    if constexpr (TYPES == GZ_E4M3E4M3F16) {
      acc = __builtin_amdgcn_mfma_f32_32x32x16_fp8_fp8(b.x, a.x, acc, 0, 0, 0);
      acc = __builtin_amdgcn_mfma_f32_32x32x16_fp8_fp8(b.y, a.y, acc, 0, 0, 0);
    } else {
      acc = __builtin_amdgcn_mfma_f32_32x32x16_bf8_bf8(b.x, a.x, acc, 0, 0, 0);
      acc = __builtin_amdgcn_mfma_f32_32x32x16_bf8_bf8(b.y, a.y, acc, 0, 0, 0);
    }
    return acc;
  } else if constexpr (TYPES == GZ_F32F32F32) {
    // 16 bytes per lane are 4 fp32 K values; v_mfma_f32_32x32x2_f32 takes one per lane (lanes 0-31: one k,
    // lanes 32-63: another), so four of them consume the fragment pair.  Full fp32 products, no tf32 rounding.
    const f32x4_t b = __builtin_bit_cast(f32x4_t, first), a = __builtin_bit_cast(f32x4_t, second);
    acc = __builtin_amdgcn_mfma_f32_32x32x2f32(b.x, a.x, acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_32x32x2f32(b.y, a.y, acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_32x32x2f32(b.z, a.z, acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_32x32x2f32(b.w, a.w, acc, 0, 0, 0);
    return acc;
  } else {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, first),
                                                   __builtin_bit_cast(bf16x8_t, second), acc, 0, 0, 0);
  }
}

// ---------------------------------------------------------------------------
// Accumulators -> D, shared by every kernel of the rung.  acc[i][j][4 q + e] of a lane is D(m, n + e) with
//   m = row0 + 32 i + lane % 32,   n = col0 + 32 j + 8 q + 4 (lane / 32)
// (row0 / col0: first row and column of the wave's sub-tile), so a lane owns four consecutive columns of one
// row.  Every index into the accumulators is a compile-time constant: written as loops, the larger epilogues
// (bf16 rounding) were not unrolled and the compiler kept all 256 accumulators in scratch memory, with a store
// after every MFMA of the main loop.
// Whole tiles, straight from the registers: one 16-byte (fp32 / int32) or 8-byte (16-bit) store per four columns.
// ---------------------------------------------------------------------------
template <int TYPES, int FM, int FN, class Acc>
__device__ __forceinline__ void store_accumulators(const GemmArgs<TYPES>& g, Acc (&acc)[FM][FN], int row0, int col0, int lane) {
  using out_t = typename Traits<TYPES>::out_t;
  const size_t LDC = (size_t)g.ldc, LDD = (size_t)g.ldd;
  const bool use_c = g.beta != 0;
  static_for<FM>([&](auto i_c) {
    constexpr int I = decltype(i_c)::value;
    const int m = row0 + 32 * I + (lane & 31);
    static_for<FN>([&](auto j_c) {
      constexpr int J = decltype(j_c)::value;
      static_for<4>([&](auto q_c) {
        constexpr int Q = decltype(q_c)::value;
        const int n = col0 + 32 * J + 8 * Q + 4 * (lane >> 5);
        const size_t o = (size_t)m * LDD + n;
        const Acc& a = acc[I][J];
        out_t cv[4] = {0, 0, 0, 0}, dv[4];
        if (use_c) __builtin_memcpy(cv, g.C + (size_t)m * LDC + n, sizeof(cv));
        dv[0] = epilogue<TYPES>(a[4 * Q + 0], g.alpha, g.beta, &cv[0]);
        dv[1] = epilogue<TYPES>(a[4 * Q + 1], g.alpha, g.beta, &cv[1]);
        dv[2] = epilogue<TYPES>(a[4 * Q + 2], g.alpha, g.beta, &cv[2]);
        dv[3] = epilogue<TYPES>(a[4 * Q + 3], g.alpha, g.beta, &cv[3]);
        __builtin_memcpy(g.D + o, dv, sizeof(dv));
      });
    });
  });
}

// The same through LDS, so that a store instruction writes whole cache lines.  Straight from the
// accumulators a wave's store covers 32 rows x 32 bytes, and the output - 64 MiB for fp32 4096^2, 256 MiB for int32
// 8192^2, written by all compute units at the same moment - left the device at about 3 TB/s (a launch with K = 64:
// 20-24 us; int8 8192 x 8192 x 128: 89 us).  Measured in interleaved runs against the direct stores, beta = 0: bf16
// 4096^3 eight waves 118.8 against 122.7 us, 8192^3 867 against 894, int8 8192^3 501 against 539; with C read as
// well (beta = 1) 136.5 against 148.9, four waves 137.1 against 135.4, int8 568 against 592.  Here each wave parks one 32-row block of its sub-tile in its own LDS
// region (row pitch COLS * 4 + 16 bytes), reads it back row by row and stores runs of COLS * sizeof(out) contiguous
// bytes (also the loads of C).  `region` is this wave's 32 x (COLS * 4 + 16) bytes; the caller has made sure that no
// wave still reads operands from LDS.
// BLK = 16: the accumulators are those of the 16x16 instructions, acc[i][j][e] = D(row0 + 16 i + lane % 16,
// col0 + 16 j + 4 (lane / 16) + e); FM and FN still count 32-row and 32-column blocks.
// TRANSPOSED (BLK = 16): the blocks come as acc[j][i], the array of a kernel that ran the transposed problem.
// BY4 (BLK = 16): within a group of 64 columns block 4 g + s holds the columns 4 c + s, c = 0 .. 15, instead of
// 16 s + c: acc[i][4 g + s][e] = D(row0 + 16 i + lane % 16, col0 + 64 g + 16 (lane / 16) + 4 e + s) - what a kernel
// ends up with that feeds the matrix instruction four consecutive columns of a row-major B per lane.  A lane's values
// of the four blocks of a group are then four consecutive columns again.
// UC: whether C is read - 2: decided here (beta != 0), 0 / 1: known to the caller.  The ragged kernels call it with a
// constant: their stores sit under each lane's own condition, and where loads of C may be pending when such a region is
// entered the compiler waits for ALL memory operations there (loads and stores return in no fixed order with respect to
// each other), i.e. for the previous store, 64 times per wave on the four-wave 256 x 256 tile (7 us per launch).
// Without loads of C nothing is waited for; with them, they are waited for once per block, before its first store.
template <int UC, int TYPES, int FM, int FN, bool RAGGED, int BLK, bool TRANSPOSED, bool BY4, class Acc, int AM, int AN>
__device__ __forceinline__ void store_accumulators_lds_impl(const GemmArgs<TYPES>& g, Acc (&acc)[AM][AN], int row0, int col0,
                                                            int lane, char* region) {
  static_assert(TRANSPOSED ? (BLK == 16 && AN == FM * 2 && AM == FN * 2)
                           : (AM == FM * (32 / BLK) && AN == FN * (32 / BLK)), "accumulator blocks of BLK x BLK");
  constexpr int NJ = TRANSPOSED ? AM : AN;   // 16-column blocks of a row
  using out_t = typename Traits<TYPES>::out_t;
  using acc_t = typename Traits<TYPES>::acc_t;
  constexpr int COLS = FN * 32, PITCH_E = COLS * 4 + 16;
  // A lane takes W consecutive columns of a row: four, or eight of a 16-bit output on whole aligned tiles, where
  // the stores are bound by their number, not their bytes (bf16 -> bf16 4096 x 4096 x 64 took 16.6 us for 32 MiB,
  // 17.7 with an fp32 output of 64 MiB).
  constexpr int W = (!RAGGED && sizeof(out_t) == 2) ? 8 : 4, WB = W * (int)sizeof(out_t);
  constexpr int LPR = COLS / W, RPI = 64 / LPR, NI = 32 / RPI;   // lanes per row, rows per instruction, instructions
  const int M = g.M, N = g.N;
  const size_t LDC = (size_t)g.ldc, LDD = (size_t)g.ldd;   // elements between the rows of C and of D
  const bool use_c = UC == 2 ? g.beta != 0 : UC == 1;
  const typename Traits<TYPES>::scalar_t beta_e = UC == 0 ? (typename Traits<TYPES>::scalar_t)0 : g.beta;   // (UC == 0: beta is 0)
  static_assert(!BY4 || (BLK == 16 && !TRANSPOSED && AN % 4 == 0), "groups of four 16-column blocks");
  char* wr = BLK == 32 ? region + (lane & 31) * PITCH_E + (lane >> 5) * 16
                       : region + (lane & 15) * PITCH_E + (lane >> 4) * (BY4 ? 64 : 16);
  const char* rd = region + (lane / LPR) * PITCH_E + (lane % LPR) * W * 4;
  const int n = col0 + (lane % LPR) * W;
  // RAGGED: M or N need not be multiples of the tile and D / C need not be aligned.  Rows and columns past the end
  // are skipped.  Where the rows of D (and C) are whole, aligned groups of four elements the stores stay vectors;
  // otherwise the block is written one element per lane with the lanes along a row, which is still whole cache
  // lines per instruction (fp16 4095 x 4097 x 63 took 65 us with four scattered 2-byte stores per lane).
  constexpr uintptr_t VEC_ALIGN = 4 * sizeof(out_t) - 1;
  const bool vec = !RAGGED || ((N & 3) == 0 && (LDD & 3) == 0 && (!use_c || (LDC & 3) == 0) &&
                               ((reinterpret_cast<uintptr_t>(g.D) | (use_c ? reinterpret_cast<uintptr_t>(g.C) : 0)) & VEC_ALIGN) == 0);
  static_for<FM>([&](auto i_c) {
    constexpr int I = decltype(i_c)::value;
    // the block's values of C first: their latency passes while the accumulators go through LDS
    out_t cv[NI][W];
    static_for<NI>([&](auto t_c) {
      constexpr int T = decltype(t_c)::value;
#pragma unroll
      for (int e = 0; e < W; e++) cv[T][e] = 0;
      // RAGGED: a lane past the last row or column reads the last row / the first columns instead (never stored).
      // The load itself is unconditional for the wave: under a lane's own condition every load ends in a merge that
      // waits for it, one load at a time.
      const int m = RAGGED ? min(row0 + 32 * I + T * RPI + lane / LPR, M - 1) : row0 + 32 * I + T * RPI + lane / LPR;
      const int nc = RAGGED ? (n < N ? n : 0) : n;
      if (use_c && vec) {
        if (g.store_hint & 2) {   // non-temporal: see mfma_store_hint
          if constexpr (WB == 16) {
            const u32x4_t w = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(g.C + (size_t)m * LDC + nc));
            __builtin_memcpy(cv[T], &w, 16);
          } else {
            const u32x2_t w = __builtin_nontemporal_load(reinterpret_cast<const u32x2_t*>(g.C + (size_t)m * LDC + nc));
            __builtin_memcpy(cv[T], &w, 8);
          }
        } else {
          __builtin_memcpy(cv[T], g.C + (size_t)m * LDC + nc, sizeof(cv[T]));
        }
      }
    });
    if constexpr (BLK == 32) {
      static_for<FN>([&](auto j_c) {
        constexpr int J = decltype(j_c)::value;
        static_for<4>([&](auto q_c) {
          constexpr int Q = decltype(q_c)::value;
          const Acc& a = acc[I][J];
          acc_t v[4] = {a[4 * Q + 0], a[4 * Q + 1], a[4 * Q + 2], a[4 * Q + 3]};
          __builtin_memcpy(wr + (32 * J + 8 * Q) * 4, v, 16);
        });
      });
    } else {
      static_for<2>([&](auto h_c) {
        constexpr int H = decltype(h_c)::value;
        static_for<NJ>([&](auto j_c) {
          constexpr int J = decltype(j_c)::value;
          if constexpr (BY4) {   // group J / 4, element J % 4 of its four blocks
            constexpr int G = J / 4, E = J % 4;
            acc_t v[4] = {acc[2 * I + H][4 * G + 0][E], acc[2 * I + H][4 * G + 1][E], acc[2 * I + H][4 * G + 2][E],
                          acc[2 * I + H][4 * G + 3][E]};
            __builtin_memcpy(wr + H * 16 * PITCH_E + (64 * G + 4 * E) * 4, v, 16);
          } else {
            const Acc& a = acc[TRANSPOSED ? J : 2 * I + H][TRANSPOSED ? 2 * I + H : J];
            acc_t v[4] = {a[0], a[1], a[2], a[3]};
            __builtin_memcpy(wr + H * 16 * PITCH_E + J * 64, v, 16);
          }
        });
      });
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    if (vec) {
      // (RAGGED: all of the block's LDS reads first - behind a lane's own condition each would be waited for on its
      // own.  Whole tiles keep read, wait and store in turn: with all reads ahead of the stores int8 8192^3 was 1.5 %
      // slower against hipBLASLt in the same process, and bf16 4096^3 no faster.)
      acc_t vs[RAGGED ? NI : 1][W];
      if constexpr (RAGGED) {
        static_for<NI>([&](auto t_c) {
          constexpr int T = decltype(t_c)::value;
          __builtin_memcpy(vs[T], rd + T * RPI * PITCH_E, W * 4);
        });
        if constexpr (UC == 1) {   // the block's values of C have arrived before the first region of a store is entered
          static_for<NI>([&](auto t_c) {
            constexpr int T = decltype(t_c)::value;
            uint32_t w[WB / 4];
            __builtin_memcpy(w, cv[T], WB);
#pragma unroll
            for (int x = 0; x < WB / 4; x++) asm volatile("" : "+v"(w[x]));
            __builtin_memcpy(cv[T], w, WB);
          });
        }
      }
      static_for<NI>([&](auto t_c) {
        constexpr int T = decltype(t_c)::value;
        acc_t v[W];
        if constexpr (RAGGED) __builtin_memcpy(v, vs[T], W * 4);
        else __builtin_memcpy(v, rd + T * RPI * PITCH_E, W * 4);
        const int m = row0 + 32 * I + T * RPI + lane / LPR;
        const size_t o = (size_t)m * LDD + n;
        if constexpr (RAGGED) {
          if (m >= M || n >= N) return;   // N is a multiple of four here: the lane's four columns end together
        }
        out_t dv[W];
        static_for<W>([&](auto e_c) {
          constexpr int E = decltype(e_c)::value;
          dv[E] = epilogue<TYPES>(v[E], g.alpha, beta_e, &cv[T][E]);
        });
        if (g.store_hint & 1) {   // non-temporal: see mfma_store_hint
          if constexpr (WB == 16) {
            u32x4_t w;
            __builtin_memcpy(&w, dv, 16);
            __builtin_nontemporal_store(w, reinterpret_cast<u32x4_t*>(g.D + o));
          } else {
            u32x2_t w;
            __builtin_memcpy(&w, dv, 8);
            __builtin_nontemporal_store(w, reinterpret_cast<u32x2_t*>(g.D + o));
          }
        } else {
          __builtin_memcpy(g.D + o, dv, sizeof(dv));
        }
      });
    } else if constexpr (RAGGED) {
      // eight rows at a time: their LDS reads first, then the stores, so that a row does not wait for the one before
      // (a sub-tile 32 columns wide: the upper half of the lanes has no column)
      constexpr int RG = 8, NC = (COLS + 63) / 64;
      const bool has_col = COLS % 64 == 0 || lane < COLS % 64;   // in the last group of 64 columns
      for (int r0 = 0; r0 < 32; r0 += RG) {
        const int mg = row0 + 32 * I + r0;
        if (mg >= M) break;
        acc_t v[RG][NC];
        static_for<RG>([&](auto r_c) {
          constexpr int R = decltype(r_c)::value;
          static_for<NC>([&](auto c_c) {
            constexpr int C = decltype(c_c)::value;
            v[R][C] = 0;
            if (C < NC - 1 || has_col) __builtin_memcpy(&v[R][C], region + (r0 + R) * PITCH_E + (C * 64 + lane) * 4, 4);
          });
        });
        static_for<RG>([&](auto r_c) {
          constexpr int R = decltype(r_c)::value;
          const int m = mg + R;
          static_for<NC>([&](auto c_c) {
            constexpr int C = decltype(c_c)::value;
            const int nn = col0 + C * 64 + lane;
            if (m < M && nn < N && (C < NC - 1 || has_col))
              g.D[(size_t)m * LDD + nn] = epilogue<TYPES>(v[R][C], g.alpha, beta_e, g.C + (size_t)m * LDC + nn);
          });
        });
      }
    }
    // No wait here: the LDS executes a wave's instructions in order, so the next block's stores, issued right
    // behind these loads, cannot overtake them, and they land while this block's values are on their way out.
    // The compiler must keep that order too (it may not see that another lane's store hits this lane's load):
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    __builtin_amdgcn_wave_barrier();
  });
}
template <int TYPES, int FM, int FN, bool RAGGED = false, int BLK = 32, bool TRANSPOSED = false, bool BY4 = false, class Acc,
          int AM, int AN>
__device__ __forceinline__ void store_accumulators_lds(const GemmArgs<TYPES>& g, Acc (&acc)[AM][AN], int row0, int col0,
                                                       int lane, char* region) {
  if constexpr (RAGGED) {
    if (g.beta != 0) store_accumulators_lds_impl<1, TYPES, FM, FN, RAGGED, BLK, TRANSPOSED, BY4>(g, acc, row0, col0, lane, region);
    else store_accumulators_lds_impl<0, TYPES, FM, FN, RAGGED, BLK, TRANSPOSED, BY4>(g, acc, row0, col0, lane, region);
  } else {
    store_accumulators_lds_impl<2, TYPES, FM, FN, RAGGED, BLK, TRANSPOSED, BY4>(g, acc, row0, col0, lane, region);
  }
}
template <int FN> constexpr int epilogue_region_bytes() { return 32 * (FN * 32 * 4 + 16); }

// MFMA instructions behind one mfma32 call
template <int TYPES> constexpr int mfmas_per_fragment() { return TYPES == GZ_F32F32F32 ? 4 : is_fp8(TYPES) ? 2 : 1; }

// 8-bit floats, the fragments of two consecutive 32-byte K steps at once: v_mfma_f32_32x32x64_f8f6f4 takes 32 bytes
// per lane and operand (format 0 = e4m3, 1 = e5m2; no block scaling).  Which k a lane's bytes stand for is the same
// on both operands.
typedef int i32x8_t __attribute__((ext_vector_type(8)));
template <int TYPES>
__device__ inline f32x16_t mfma_f8_pair(u32x4_t first0, u32x4_t first1, u32x4_t second0, u32x4_t second1, f32x16_t acc) {
  const i32x8_t f = __builtin_bit_cast(i32x8_t, __builtin_shufflevector(first0, first1, 0, 1, 2, 3, 4, 5, 6, 7));
  const i32x8_t s = __builtin_bit_cast(i32x8_t, __builtin_shufflevector(second0, second1, 0, 1, 2, 3, 4, 5, 6, 7));
  constexpr int FMT = TYPES == GZ_E5M2E5M2F16 ? 1 : 0;
  return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(f, s, acc, FMT, FMT, 0, 0, 0, 0);
}

constexpr int SLAB_BYTES = 128;           // K bytes per tile row per slab
constexpr int PITCH = SLAB_BYTES + 16;    // LDS row pitch
constexpr int KSTEPS = SLAB_BYTES / 32;   // MFMA steps per slab

// 16-byte global load of `EPV` elements starting at element (line, pos) of a
// matrix whose lines are `extent` long and `pitch` elements apart.  With EDGE the access is predicated and
// zero-filled, and may be unaligned (gfx950 global loads tolerate that).
template <typename in_t, bool EDGE>
__device__ inline u32x4_t load16(const in_t* __restrict__ base, int line, int lines, int pos, int extent, size_t pitch) {
  constexpr int EPV = 16 / (int)sizeof(in_t);
  if constexpr (!EDGE) {
    return *reinterpret_cast<const u32x4_t*>(base + (size_t)line * pitch + pos);
  } else {
    u32x4_t v = {0u, 0u, 0u, 0u};
    if (line < lines) {
      const in_t* p = base + (size_t)line * pitch + pos;
      if (pos + EPV <= extent) {
        __builtin_memcpy(&v, p, 16);
      } else if (pos < extent) {
        in_t tmp[EPV];
#pragma unroll
        for (int e = 0; e < EPV; e++) tmp[e] = (pos + e < extent) ? p[e] : (in_t)0;
        __builtin_memcpy(&v, tmp, 16);
      }
    }
    return v;
  }
}

// Scheduling hint for the region it closes: spread N_OTHER instructions of class MASK (0x020 global loads, 0x200 LDS
// stores) evenly between the region's N_MFMA MFMAs instead of leaving them in one block.
template <int MASK, int N_OTHER, int N_MFMA> __device__ inline void mix_into_mfmas() {
  if constexpr (N_OTHER >= N_MFMA) {
    constexpr int PER = (N_OTHER + N_MFMA - 1) / N_MFMA;
#pragma unroll
    for (int x = 0; x < N_MFMA; x++) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(MASK, PER, 0);
    }
  } else {
    constexpr int PER = N_MFMA / N_OTHER;
#pragma unroll
    for (int x = 0; x < N_OTHER; x++) {
      __builtin_amdgcn_sched_group_barrier(0x008, PER, 0);
      __builtin_amdgcn_sched_group_barrier(MASK, 1, 0);
    }
  }
}

// The same for two classes at once: N_ST LDS stores, then N_LD global loads, after each MFMA its share of both.
template <int N_ST, int N_LD, int N_MFMA> __device__ inline void mix2_into_mfmas() {
  constexpr int PER_ST = (N_ST + N_MFMA - 1) / N_MFMA, PER_LD = (N_LD + N_MFMA - 1) / N_MFMA;
#pragma unroll
  for (int x = 0; x < N_MFMA; x++) {
    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
    __builtin_amdgcn_sched_group_barrier(0x200, PER_ST, 0);
    __builtin_amdgcn_sched_group_barrier(0x020, PER_LD, 0);
  }
}

// ---------------------------------------------------------------------------
// Slab staging: global -> registers -> LDS.
// KC == true : operand lines are K-contiguous (row-major A, column-major B).
//              chunk = 16 B of one tile row.
// KC == false: operand lines run along M/N (column-major A, row-major B).
//              unit = TR k-lines x 16 B; transposed to EPV dwords of TR k-values.
// ---------------------------------------------------------------------------
template <typename in_t, int ROWS, int NT, bool KC, bool EDGE> struct Stager {
  static constexpr int ES = (int)sizeof(in_t);
  static constexpr int EPV = 16 / ES;
  static constexpr int BK = SLAB_BYTES / ES;
  static constexpr int TR = 4 / ES;  // k-lines packed per LDS dword
  // KC: ROWS*8 chunks ; !KC: (BK/TR)*(ROWS/EPV) units of TR vectors
  static constexpr int VECS = ROWS * 8 / NT;  // 16-byte vectors per thread (same either way)
  static constexpr int UNITS = VECS / TR;
  static_assert(ROWS * 8 % NT == 0, "tile rows must divide over the work-group");
  static_assert(KC || (VECS % TR == 0 && VECS >= TR), "transposing stager needs whole units");

  u32x4_t r[VECS];

  // Transposing case: which 16-byte column (mc) of which k unit (ku) a thread moves. Within a wavefront MC_LO
  // neighbouring lanes take one contiguous run of a k line (whole 64- or 128-byte segments of global memory) and
  // the other lane bits walk over k units, so that the dword stores of one instruction, which land EPV * PITCH
  // bytes apart per column step, spread over the LDS banks through their k offset instead of piling onto a few.
  // 32-bit elements are not transposed at all: a k line of the tile goes to LDS as it lies in memory (NAT_PITCH
  // bytes per k line, lanes along the line), and the fragment reads gather one dword per k value instead.
  static constexpr int MC_LO = 4;
  static constexpr int NAT_PITCH = ROWS * 4 + 32;
  __device__ static inline void unit_of(int id, int& mc, int& ku) {
    constexpr int MC = ROWS / EPV;
    if constexpr (ES == 4) {
      mc = id % MC;
      ku = id / MC;
    } else {
      constexpr int KU_LO = 64 / MC_LO, MC_HI = MC / MC_LO;
      static_assert(MC % MC_LO == 0 && NT % 64 == 0, "unit mapping works on whole wavefronts");
      const int hi = id >> 6;
      mc = (id % MC_LO) + (hi % MC_HI) * MC_LO;
      ku = (id & 63) / MC_LO + (hi / MC_HI) * KU_LO;
    }
  }
  // LDS store instructions of one store() call
  static constexpr int LDS_STORES = KC ? VECS : ES == 4 ? UNITS : UNITS * EPV;
  // bytes of one staged slab of this operand
  static constexpr int LDS_BYTES = (!KC && ES == 4) ? BK * NAT_PITCH : ROWS * PITCH;

  // rows_total: M or N ; row0: first tile row ; k0: first k of the slab ; pitch: the operand's leading dimension
  // (elements between its lines: tile rows of a K-contiguous operand, k lines of one whose lines run along M / N)
  // The same for a slab whose k lines lie inside the matrix: k0 + BK <= K.  Every load is unconditional.  Lines of
  // the tile past the last row or column of the matrix are read from the last one instead: what is computed from
  // them is never stored, so it may be anything.  An operand whose lines run along M / N reads a 16-byte piece that
  // reaches past the end of its k line as it lies in memory, i.e. into the start of the next k line: such a tile's
  // slab must not hold the last k line of the matrix (k0 + BK <= K - 1).  The predicated loads of load() each end in a merge of
  // the loaded value with zero, and the compiler waits for a load at such a merge: eight loads per slab, one after
  // the other behind eight waits (fp16 4095 x 4096 x 1023 row/row: 57 us, of which the waits were a third).
  __device__ inline void load_inside(const in_t* __restrict__ base, int rows_total, int K, int row0, int k0, int tid, size_t pitch) {
    if constexpr (KC) {
#pragma unroll
      for (int it = 0; it < VECS; it++) {
        const int id = it * NT + tid;
        const int row = min(row0 + (id >> 3), rows_total - 1), c = id & 7;
        __builtin_memcpy(&r[it], base + (size_t)row * pitch + k0 + c * EPV, 16);
      }
    } else {
#pragma unroll
      for (int u = 0; u < UNITS; u++) {
        int mc, ku;
        unit_of(u * NT + tid, mc, ku);
#pragma unroll
        for (int t = 0; t < TR; t++)
          __builtin_memcpy(&r[u * TR + t], base + (size_t)(k0 + ku * TR + t) * pitch + min(row0 + mc * EPV, rows_total - 1), 16);
      }
    }
  }
  __device__ inline void load(const in_t* __restrict__ base, int rows_total, int K, int row0, int k0, int tid, size_t pitch) {
    if constexpr (KC) {
#pragma unroll
      for (int it = 0; it < VECS; it++) {
        const int id = it * NT + tid;
        const int row = id >> 3, c = id & 7;
        r[it] = load16<in_t, EDGE>(base, row0 + row, rows_total, k0 + c * EPV, K, pitch);
      }
    } else {
#pragma unroll
      for (int u = 0; u < UNITS; u++) {
        int mc, ku;
        unit_of(u * NT + tid, mc, ku);
#pragma unroll
        for (int t = 0; t < TR; t++)
          r[u * TR + t] = load16<in_t, EDGE>(base, k0 + ku * TR + t, K, row0 + mc * EPV, rows_total, pitch);
      }
    }
  }

  __device__ inline void store(char* lds, int tid) const {
    if constexpr (KC) {
#pragma unroll
      for (int it = 0; it < VECS; it++) {
        const int id = it * NT + tid;
        const int row = id >> 3, c = id & 7;
        *reinterpret_cast<u32x4_t*>(lds + row * PITCH + c * 16) = r[it];
      }
    } else {
#pragma unroll
      for (int u = 0; u < UNITS; u++) {
        int mc, ku;
        unit_of(u * NT + tid, mc, ku);
        char* dst = lds + (mc * EPV) * PITCH + ku * 4;
        if constexpr (ES == 4) {  // one k-line per unit, kept as it is
          *reinterpret_cast<u32x4_t*>(lds + ku * NAT_PITCH + mc * 16) = r[u];
        } else if constexpr (ES == 2) {
          const u32x4_t lo = r[u * 2], hi = r[u * 2 + 1];
#pragma unroll
          for (int w = 0; w < 4; w++) {
            // elements 2w and 2w+1 of both k-lines
            const uint32_t e0 = __builtin_amdgcn_perm(hi[w], lo[w], 0x05040100u);  // lo.lo16 | hi.lo16<<16
            const uint32_t e1 = __builtin_amdgcn_perm(hi[w], lo[w], 0x07060302u);  // lo.hi16 | hi.hi16<<16
            *reinterpret_cast<uint32_t*>(dst + (2 * w) * PITCH) = e0;
            *reinterpret_cast<uint32_t*>(dst + (2 * w + 1) * PITCH) = e1;
          }
        } else {
          const u32x4_t v0 = r[u * 4], v1 = r[u * 4 + 1], v2 = r[u * 4 + 2], v3 = r[u * 4 + 3];
#pragma unroll
          for (int w = 0; w < 4; w++) {
            // 4x4 byte transpose of {v0[w], v1[w], v2[w], v3[w]}
            const uint32_t a01_lo = __builtin_amdgcn_perm(v1[w], v0[w], 0x05010400u);  // v0.b0 v1.b0 v0.b1 v1.b1
            const uint32_t a01_hi = __builtin_amdgcn_perm(v1[w], v0[w], 0x07030602u);  // v0.b2 v1.b2 v0.b3 v1.b3
            const uint32_t a23_lo = __builtin_amdgcn_perm(v3[w], v2[w], 0x05010400u);
            const uint32_t a23_hi = __builtin_amdgcn_perm(v3[w], v2[w], 0x07030602u);
            const uint32_t e0 = __builtin_amdgcn_perm(a23_lo, a01_lo, 0x05040100u);
            const uint32_t e1 = __builtin_amdgcn_perm(a23_lo, a01_lo, 0x07060302u);
            const uint32_t e2 = __builtin_amdgcn_perm(a23_hi, a01_hi, 0x05040100u);
            const uint32_t e3 = __builtin_amdgcn_perm(a23_hi, a01_hi, 0x07060302u);
            *reinterpret_cast<uint32_t*>(dst + (4 * w + 0) * PITCH) = e0;
            *reinterpret_cast<uint32_t*>(dst + (4 * w + 1) * PITCH) = e1;
            *reinterpret_cast<uint32_t*>(dst + (4 * w + 2) * PITCH) = e2;
            *reinterpret_cast<uint32_t*>(dst + (4 * w + 3) * PITCH) = e3;
          }
        }
      }
    }
  }
};

// Work-group id -> tile.  Work-groups are dealt round-robin to the 8 XCDs, each
// with a private L2; give every XCD a contiguous run of logical tile ids and
// walk those in bands of GROUP_M tile-rows so that an XCD's tiles share A rows
// and B columns.
// (lid_of_block: which logical tile id of `total` launched ones a work-group takes; tile_of_lid: where that id
// lies in the grid of tiles.)
__device__ inline int lid_of_block(int bid, int total) {
  constexpr int XCDS = 8;
  const int per = total / XCDS, rem = total % XCDS;
  const int xcd = bid % XCDS, idx = bid / XCDS;
  return xcd * per + (xcd < rem ? xcd : rem) + idx;
}
__device__ inline void tile_of_lid(int lid, int tiles_m, int tiles_n, int& tm, int& tn) {
  constexpr int GROUP_M = 4;
  const int band = GROUP_M * tiles_n;
  const int b = lid / band;
  const int first_m = b * GROUP_M;
  const int rows = (tiles_m - first_m) < GROUP_M ? (tiles_m - first_m) : GROUP_M;
  const int in_band = lid - b * band;
  tm = first_m + in_band % rows;
  tn = in_band / rows;
}
__device__ inline void tile_of_block(int bid, int tiles_m, int tiles_n, int& tm, int& tn) {
  tile_of_lid(lid_of_block(bid, tiles_m * tiles_n), tiles_m, tiles_n, tm, tn);
}

template <int TYPES, int BM, int BN, int WAVES_M, int WAVES_N, bool A_KC, bool B_KC, bool EDGE>
__global__ void __launch_bounds__(WAVES_M* WAVES_N * 64)
    mfma_gemm_kernel(GemmArgs<TYPES> g, int tiles_m, int tiles_n) {
  using T = Traits<TYPES>;
  using in_t = typename T::in_t;
  using acc_v = typename AccVec<TYPES>::type;
  constexpr int NT = WAVES_M * WAVES_N * 64;
  constexpr int ES = (int)sizeof(in_t);
  constexpr int BK = SLAB_BYTES / ES;
  constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;
  constexpr int FM = WM / 32, FN = WN / 32;
  static_assert(WM % 32 == 0 && WN % 32 == 0, "wave tile must be a multiple of the 32x32 MFMA block");
  using StagerA = Stager<in_t, BM, NT, A_KC, EDGE>;
  using StagerB = Stager<in_t, BN, NT, B_KC, EDGE>;
  constexpr bool A_NAT = ES == 4 && !A_KC, B_NAT = ES == 4 && !B_KC;  // k lines kept whole in LDS
  constexpr int A_BYTES = StagerA::LDS_BYTES, B_BYTES = StagerB::LDS_BYTES;
  constexpr int STAGE_BYTES = A_BYTES + B_BYTES;

  extern __shared__ __attribute__((aligned(16))) char lds[];

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int wm = wave % WAVES_M, wn = wave / WAVES_M;
  int tm, tn;
  tile_of_block(blockIdx.x, tiles_m, tiles_n, tm, tn);
  const int m0 = tm * BM, n0 = tn * BN;

  StagerA sa;
  StagerB sb;
  // The 64 x 64 tile has so few matrix instructions per slab (sixteen per wave) that a slab asked for one iteration
  // ahead has not arrived when its turn comes, and a work-group that is alone on its compute unit waits for it in
  // every iteration: it keeps TWO slabs in flight, in two sets of registers that take turns.
  constexpr bool DEEP = BM == 64 && BN == 64;
  constexpr int LEAD = DEEP ? 3 : 2;   // a slab is asked for LEAD iterations before it is multiplied
  StagerA sa2;
  StagerB sb2;

  acc_v acc[FM][FN];
#pragma unroll
  for (int i = 0; i < FM; i++)
#pragma unroll
    for (int j = 0; j < FN; j++)
#pragma unroll
      for (int v = 0; v < 16; v++) acc[i][j][v] = 0;

  const int ktiles = (g.K + BK - 1) / BK;

  // fragment base offsets of this lane inside a stage
  const int frag_row = lane & 31, frag_k = (lane >> 5) * 16;
  // (a whole-k-line operand: k value (lane / 32) * 4 + e of a step lies e lines further down, at this lane's row)
  const int a_off = A_NAT ? (lane >> 5) * 4 * StagerA::NAT_PITCH + (wm * WM + frag_row) * 4
                          : (wm * WM + frag_row) * PITCH + frag_k;
  const int b_off = A_BYTES + (B_NAT ? (lane >> 5) * 4 * StagerB::NAT_PITCH + (wn * WN + frag_row) * 4
                                     : (wn * WN + frag_row) * PITCH + frag_k);

  // Two fragment sets: while the MFMAs of one K step run, the ds_reads of the next are in flight.  (8-bit floats:
  // two pairs of sets, a pair holds two consecutive K steps for one 64-deep MFMA.)
  constexpr bool F8 = is_fp8(TYPES);
  u32x4_t af[F8 ? 4 : 2][FM], bf[F8 ? 4 : 2][FN];
  auto read_frags = [&](int set, const char* stage, int ks) {
#pragma unroll
    for (int i = 0; i < FM; i++) {
      if constexpr (A_NAT) {
        const char* p = stage + a_off + ks * 8 * StagerA::NAT_PITCH + i * 32 * 4;
        af[set][i] = u32x4_t{*reinterpret_cast<const uint32_t*>(p),
                             *reinterpret_cast<const uint32_t*>(p + StagerA::NAT_PITCH),
                             *reinterpret_cast<const uint32_t*>(p + 2 * StagerA::NAT_PITCH),
                             *reinterpret_cast<const uint32_t*>(p + 3 * StagerA::NAT_PITCH)};
      } else {
        af[set][i] = *reinterpret_cast<const u32x4_t*>(stage + a_off + i * 32 * PITCH + ks * 32);
      }
    }
#pragma unroll
    for (int j = 0; j < FN; j++) {
      if constexpr (B_NAT) {
        const char* p = stage + b_off + ks * 8 * StagerB::NAT_PITCH + j * 32 * 4;
        bf[set][j] = u32x4_t{*reinterpret_cast<const uint32_t*>(p),
                             *reinterpret_cast<const uint32_t*>(p + StagerB::NAT_PITCH),
                             *reinterpret_cast<const uint32_t*>(p + 2 * StagerB::NAT_PITCH),
                             *reinterpret_cast<const uint32_t*>(p + 3 * StagerB::NAT_PITCH)};
      } else {
        bf[set][j] = *reinterpret_cast<const u32x4_t*>(stage + b_off + j * 32 * PITCH + ks * 32);
      }
    }
  };
  auto mma = [&](int set) {
#pragma unroll
    for (int i = 0; i < FM; i++)
#pragma unroll
      for (int j = 0; j < FN; j++) acc[i][j] = mfma32<TYPES>(bf[set][j], af[set][i], acc[i][j]);
  };

  // A slab of the edge kernels is loaded without predication where its k lines lie inside the matrix
  // (Stager::load_inside): whole slabs of K; on a tile that reaches past the end of an M- or N-contiguous operand's
  // lines, whole slabs before the last k line.  The same for all lanes.
  // The lambdas are inlined by force: left to itself the compiler makes calls of them in the four-wave instances,
  // with both stagers in scratch memory.
  constexpr bool PEEL = EDGE;
  const bool ragged_lines = (!A_KC && m0 + BM > g.M) || (!B_KC && n0 + BN > g.N);
  // (lines shorter than a 16-byte piece: a piece could reach further than the next k line, so no such slabs)
  const bool short_lines = (!A_KC && g.lda < 16) || (!B_KC && g.ldb < 16);
  const int full_slabs = ragged_lines ? (short_lines ? 0 : (g.K - 1) / BK) : g.K / BK;
  // how a slab is loaded: predicated, unconditionally (inside), or not at all (the last two iterations of the edge
  // kernels have no slab left to ask for; the registers keep what they hold and what is stored from them is never read)
  using LoadPredicated = std::integral_constant<int, 0>;
  using LoadInside = std::integral_constant<int, 1>;
  using LoadNothing = std::integral_constant<int, 2>;
  auto load_slab = [&](auto mode_c, int k0, StagerA& xa, StagerB& xb) __attribute__((always_inline)) {
    constexpr int MODE = decltype(mode_c)::value;
    if constexpr (MODE == 1) {
      xa.load_inside(g.A, g.M, g.K, m0, k0, tid, (size_t)g.lda);
      xb.load_inside(g.B, g.N, g.K, n0, k0, tid, (size_t)g.ldb);
    } else if constexpr (MODE == 0) {
      xa.load(g.A, g.M, g.K, m0, k0, tid, (size_t)g.lda);
      xb.load(g.B, g.N, g.K, n0, k0, tid, (size_t)g.ldb);
    }
  };
  auto load_slab_checked = [&](int slab, StagerA& xa, StagerB& xb) __attribute__((always_inline)) {
    if constexpr (PEEL) {
      if (slab < full_slabs) {
        load_slab(LoadInside{}, slab * BK, xa, xb);
        return;
      }
    }
    load_slab(LoadPredicated{}, slab * BK, xa, xb);
  };
  // Prologue: slab 0 into LDS, slab 1 parked in registers (DEEP: and slab 2 in the second set), fragments of
  // (slab 0, step 0) requested.
  load_slab_checked(0, sa, sb);
  sa.store(lds, tid);
  sb.store(lds + A_BYTES, tid);
  if (ktiles > 1) load_slab_checked(1, sa, sb);
  if constexpr (DEEP) {
    if (ktiles > 2) load_slab_checked(2, sa2, sb2);
  }
  __syncthreads();
  read_frags(0, lds, 0);
  // iterations whose loads (slab kt + LEAD) are inside: the first kt_inside of them
  const int kt_inside = PEEL ? max(0, min(ktiles, full_slabs - LEAD)) : 0;
  // iteration kt parks slab kt + 1 from the register set of its parity (the only set unless DEEP) and refills it
  using Set0 = std::integral_constant<int, 0>;
  using Set1 = std::integral_constant<int, 1>;
  auto run_iters = [&](auto&& iter, auto mode_c, int& kt, int end) __attribute__((always_inline)) {
    if constexpr (!DEEP) {
      for (; kt < end; kt++) iter(mode_c, Set0{}, kt);
    } else {
      if ((kt & 1) && kt < end) {
        iter(mode_c, Set1{}, kt);
        kt++;
      }
      for (; kt + 1 < end; kt += 2) {
        iter(mode_c, Set0{}, kt);
        iter(mode_c, Set1{}, kt + 1);
      }
      if (kt < end) {
        iter(mode_c, Set0{}, kt);
        kt++;
      }
    }
  };

  // Steady state per slab (KSTEPS = 4 MFMA steps), one barrier per slab:
  //   step 0 : request step 1's fragments; the parked registers (slab kt+1) go to the other LDS buffer, which every
  //            wave left before the previous barrier, one store between every few MFMAs
  //   step 1 : request step 2's fragments; slab kt+2 is requested from global memory, again between the MFMAs
  //   step 2 : request step 3's fragments
  //   barrier: every wave has written the other buffer and has its last fragments of this one
  //   step 3 : request (slab kt+1, step 0) fragments from the other buffer
  // A wave that issues its stores and loads in one block leaves the matrix pipe idle meanwhile (it holds only a few
  // MFMAs ahead), and all waves of the work-group would do so at the same time. The loop body is one straight line:
  // past the end of K the predicated loads of the edge kernels fetch nothing, the others fetch the last slab again,
  // and what is parked in LDS then is never read.
  static_assert(KSTEPS == 4, "the slab loop is written out for four steps");
  constexpr int MFMAS_PER_STEP = FM * FN * mfmas_per_fragment<TYPES>();
  if constexpr (F8) {
    // 8-bit floats: the same loop in two double steps, each one v_mfma_f32_32x32x64_f8f6f4 per 32x32 block
    auto mma2 = [&](int pair) {
#pragma unroll
      for (int i = 0; i < FM; i++)
#pragma unroll
        for (int j = 0; j < FN; j++)
          acc[i][j] = mfma_f8_pair<TYPES>(bf[2 * pair][j], bf[2 * pair + 1][j], af[2 * pair][i], af[2 * pair + 1][i], acc[i][j]);
    };
    read_frags(1, lds, 1);
    auto slab_iter = [&](auto mode_c, auto set_c, int kt) __attribute__((always_inline)) {
      const char* cur = lds + (kt & 1) * STAGE_BYTES;
      char* nxt = lds + ((kt + 1) & 1) * STAGE_BYTES;
      StagerA& xa = [&]() -> StagerA& { if constexpr (decltype(set_c)::value) return sa2; else return sa; }();
      StagerB& xb = [&]() -> StagerB& { if constexpr (decltype(set_c)::value) return sb2; else return sb; }();
      read_frags(2, cur, 2);
      read_frags(3, cur, 3);
      xa.store(nxt, tid);
      xb.store(nxt + A_BYTES, tid);
      load_slab(mode_c, (EDGE || kt + LEAD < ktiles ? kt + LEAD : ktiles - 1) * BK, xa, xb);
      mma2(0);
      mix2_into_mfmas<StagerA::LDS_STORES + StagerB::LDS_STORES, StagerA::VECS + StagerB::VECS, FM * FN>();
      __builtin_amdgcn_sched_barrier(0);

      __syncthreads();
      read_frags(0, nxt, 0);
      read_frags(1, nxt, 1);
      mma2(1);
      __builtin_amdgcn_sched_barrier(0);
    };
    int kt = 0;
    if constexpr (PEEL) run_iters(slab_iter, LoadInside{}, kt, kt_inside);
    run_iters(slab_iter, LoadPredicated{}, kt, PEEL ? ktiles - LEAD : ktiles);
    if constexpr (PEEL) run_iters(slab_iter, LoadNothing{}, kt, ktiles);
  } else {
    auto slab_iter = [&](auto mode_c, auto set_c, int kt) __attribute__((always_inline)) {
      const char* cur = lds + (kt & 1) * STAGE_BYTES;
      char* nxt = lds + ((kt + 1) & 1) * STAGE_BYTES;
      StagerA& xa = [&]() -> StagerA& { if constexpr (decltype(set_c)::value) return sa2; else return sa; }();
      StagerB& xb = [&]() -> StagerB& { if constexpr (decltype(set_c)::value) return sb2; else return sb; }();

      read_frags(1, cur, 1);
      xa.store(nxt, tid);
      xb.store(nxt + A_BYTES, tid);
      load_slab(mode_c, (EDGE || kt + LEAD < ktiles ? kt + LEAD : ktiles - 1) * BK, xa, xb);
      mma(0);
      mix2_into_mfmas<StagerA::LDS_STORES + StagerB::LDS_STORES, StagerA::VECS + StagerB::VECS, MFMAS_PER_STEP>();
      __builtin_amdgcn_sched_barrier(0);

      read_frags(0, cur, 2);
      mma(1);
      __builtin_amdgcn_sched_barrier(0);

      read_frags(1, cur, 3);
      mma(0);
      __builtin_amdgcn_sched_barrier(0);

      __syncthreads();
      read_frags(0, nxt, 0);
      mma(1);
      __builtin_amdgcn_sched_barrier(0);
    };
    int kt = 0;
    if constexpr (PEEL) run_iters(slab_iter, LoadInside{}, kt, kt_inside);
    run_iters(slab_iter, LoadPredicated{}, kt, PEEL ? ktiles - LEAD : ktiles);
    if constexpr (PEEL) run_iters(slab_iter, LoadNothing{}, kt, ktiles);
  }

  static_assert(NT / 64 * epilogue_region_bytes<FN>() <= 2 * STAGE_BYTES, "the epilogue reuses the operand buffers");
  __syncthreads();   // every wave has its last fragments: the operand buffers are free
  store_accumulators_lds<TYPES, FM, FN, EDGE>(g, acc, m0 + wm * WM, n0 + wn * WN, lane, lds + wave * epilogue_region_bytes<FN>());
}

// ---------------------------------------------------------------------------
// Fast path: both operands K-contiguous, whole tiles, 16-byte aligned.
//
// Global memory is copied straight into LDS by global_load_lds_dwordx4 (no
// staging registers, no ds_write): one wave instruction moves 8 tile rows x 128
// bytes and the hardware lays the 64 lanes' 16-byte chunks down contiguously, so
// LDS rows are unpadded.  Bank conflicts are avoided by permuting which global
// chunk each lane fetches: chunk c of tile row r lives at position
//     p = c ^ swz(r),   swz(r) = (r & 7) ^ ((r >> 3) & 1)
// which spreads any 8 consecutive rows over the 8 chunk columns and any 16
// consecutive rows over both 128-byte halves of a 64-bank line.
// ---------------------------------------------------------------------------
__device__ inline int dtl_swz(int r) { return (r & 7) ^ ((r >> 3) & 1); }

typedef __attribute__((address_space(1))) const void* gptr_t;
typedef __attribute__((address_space(3))) void* lptr_t;

// 16-byte piece c of K row r of a row-major B slab is stored at position c ^ dtl_tr_swz(r): a transposing read of
// a 32-column block touches 4 K rows x 64 bytes (16-bit) or 8 K rows x 32 bytes (int8), and the rows of a slab are
// a whole number of (or half a) 256-byte bank lines apart, so without this they would all hit the same banks.
template <int ES, int PIECES_PER_ROW> __device__ inline int dtl_tr_swz(int r) {
  static_assert(PIECES_PER_ROW >= 16 || (ES == 1 && PIECES_PER_ROW == 8), "row too short for the swizzle");
  if constexpr (ES == 2) return (r & 3) << 2;
  else if constexpr (PIECES_PER_ROW >= 16) return (r & 7) << 1;
  else return ((r >> 1) & 3) << 1;
}
typedef short s16x4_t __attribute__((ext_vector_type(4)));
typedef int i32x2_t __attribute__((ext_vector_type(2)));
// half a fragment through ds_read_b64_tr_b16 / ds_read_b64_tr_b8: lane i of 16 addresses 8 bytes of a [4 x 16]
// ([8 x 16]) block, row by row, and receives column i
template <int ES> __device__ inline u32x2_t lds_read_tr(const char* p) {
  if constexpr (ES == 2)
    return __builtin_bit_cast(u32x2_t, __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4_t*)p));
  else
    return __builtin_bit_cast(u32x2_t, __builtin_amdgcn_ds_read_tr8_b64_v2i32((__attribute__((address_space(3))) i32x2_t*)p));
}

template <int TYPES, int BM, int BN, int WAVES_M, int WAVES_N, bool B_KC = true>
__global__ void __launch_bounds__(WAVES_M* WAVES_N * 64)
    mfma_dtl_kernel(GemmArgs<TYPES> g, int tiles_m, int tiles_n) {
  using T = Traits<TYPES>;
  using in_t = typename T::in_t;
  using acc_v = typename AccVec<TYPES>::type;
  constexpr int NW = WAVES_M * WAVES_N;
  constexpr int ES = (int)sizeof(in_t);
  constexpr int EPV = 16 / ES;
  constexpr int BK = SLAB_BYTES / ES;
  constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;
  constexpr int FM = WM / 32, FN = WN / 32;
  constexpr int ROWB = SLAB_BYTES;  // unpadded LDS row
  constexpr int A_BYTES = BM * ROWB, B_BYTES = BN * ROWB;
  constexpr int STAGE_BYTES = A_BYTES + B_BYTES;
  constexpr int A_PW = BM / 8 / NW, B_PW = BN / 8 / NW;  // 1 KiB copy instructions per wave and slab
  static_assert(BM % (8 * NW) == 0 && BN % (8 * NW) == 0, "tile rows must divide over the waves");

  extern __shared__ __attribute__((aligned(1024))) char lds[];

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int wm = wave % WAVES_M, wn = wave / WAVES_M;
  int tm, tn;
  tile_of_block(blockIdx.x, tiles_m, tiles_n, tm, tn);
  const int m0 = tm * BM, n0 = tn * BN;
  const int K = g.K;

  // ---- copy addressing: lane -> (row lr of an 8-row group, LDS position lp) ----
  const int lr = lane >> 3, lp = lane & 7;
  // the 8-row group index q = wave*PW + t has the parity of t when PW is even; (wave*PW)&1 covers odd PW
  const in_t* a_src[2];
  const in_t* b_src[2];
  // row-major B: the slab is BK K rows of BN elements; a copy moves KRC whole rows, LPR lanes per row
  constexpr int TR_PITCH = BN * ES, KRC = 1024 / TR_PITCH, LPR = 64 / KRC, PPR = TR_PITCH / 16;
  const size_t LDA = (size_t)g.lda, LDB = (size_t)g.ldb;
#pragma unroll
  for (int par = 0; par < 2; par++) {
    const int ca = lp ^ lr ^ (((wave * A_PW) & 1) ^ par);
    const int cb = lp ^ lr ^ (((wave * B_PW) & 1) ^ par);
    a_src[par] = g.A + (size_t)(m0 + 8 * wave * A_PW + lr) * LDA + ca * EPV;
    if constexpr (B_KC) {
      b_src[par] = g.B + (size_t)(n0 + 8 * wave * B_PW + lr) * LDB + cb * EPV;
    } else {
      static_assert(B_KC || (KRC >= 4 && KRC * TR_PITCH == 1024), "the swizzle of a row must not depend on the copy index");
      const int kr = lane / LPR;  // row within the copy; rows of a copy start at a multiple of KRC >= 4 (8 for int8)
      b_src[par] = g.B + (size_t)(wave * B_PW * KRC + kr) * LDB + n0 + ((lane % LPR) ^ dtl_tr_swz<ES, PPR>(kr)) * EPV;
    }
  }
  auto copy_slab = [&](char* stage, int k0) {
#pragma unroll
    for (int t = 0; t < A_PW; t++)
      __builtin_amdgcn_global_load_lds((gptr_t)(a_src[t & 1] + (size_t)(8 * t) * LDA + k0),
                                       (lptr_t)(stage + (wave * A_PW + t) * 1024), 16, 0, 0);
#pragma unroll
    for (int t = 0; t < B_PW; t++) {
      if constexpr (B_KC)
        __builtin_amdgcn_global_load_lds((gptr_t)(b_src[t & 1] + (size_t)(8 * t) * LDB + k0),
                                         (lptr_t)(stage + A_BYTES + (wave * B_PW + t) * 1024), 16, 0, 0);
      else
        __builtin_amdgcn_global_load_lds((gptr_t)(b_src[0] + (size_t)(k0 + KRC * t) * LDB),
                                         (lptr_t)(stage + A_BYTES + (wave * B_PW + t) * 1024), 16, 0, 0);
    }
  };

  // ---- fragment addressing ----
  const int frag_row = lane & 31, half = lane >> 5;
  const int sw = dtl_swz(frag_row);
  int pos[KSTEPS];
#pragma unroll
  for (int ks = 0; ks < KSTEPS; ks++) pos[ks] = ((ks * 2 + half) ^ sw) * 16;
  const int a_base = (wm * WM + frag_row) * ROWB;
  const int b_base = A_BYTES + (wn * WN + frag_row) * ROWB;

  acc_v acc[FM][FN];
#pragma unroll
  for (int i = 0; i < FM; i++)
#pragma unroll
    for (int j = 0; j < FN; j++)
#pragma unroll
      for (int v = 0; v < 16; v++) acc[i][j][v] = 0;

  // transposing reads of a row-major B slab: lane i of a 16-lane group addresses K row fi of the block's rows and the
  // 8 bytes holding columns 16 (group & 1) + (4 or 8) (i % lanes-per-row); groups 2, 3 take the upper half of the step
  constexpr int TR_LPR = ES == 2 ? 4 : 2;
  constexpr int TR_STEP_ROWS = 32 / ES;         // K rows per MFMA step: 16 (16-bit) or 32 (int8)
  constexpr int TR_HALF_ROWS = 16 / TR_LPR;     // K rows per transposing read: 4 or 8
  int tr_off[FN];
  if constexpr (!B_KC) {
    const int i16 = lane & 15, fi = i16 / TR_LPR;
    const int n_sub = ((lane >> 4) & 1) * 16 + (i16 % TR_LPR) * (8 / ES);
    const int krow = (lane >> 5) * (TR_STEP_ROWS / 2) + fi;
#pragma unroll
    for (int j = 0; j < FN; j++) {
      const int n_local = wn * WN + j * 32 + n_sub;
      tr_off[j] = A_BYTES + krow * TR_PITCH + (((n_local / EPV) ^ dtl_tr_swz<ES, PPR>(fi)) * 16) + (n_local % EPV) * ES;
    }
  }
  constexpr bool F8 = is_fp8(TYPES);  // two pairs of fragment sets, a pair feeds one 64-deep MFMA per block
  u32x4_t af[F8 ? 4 : 2][FM], bf[F8 ? 4 : 2][FN];
  auto read_frags = [&](int set, const char* stage, int ks) {
#pragma unroll
    for (int i = 0; i < FM; i++)
      af[set][i] = *reinterpret_cast<const u32x4_t*>(stage + a_base + i * 32 * ROWB + pos[ks]);
#pragma unroll
    for (int j = 0; j < FN; j++) {
      if constexpr (B_KC) {
        bf[set][j] = *reinterpret_cast<const u32x4_t*>(stage + b_base + j * 32 * ROWB + pos[ks]);
      } else {
        const char* p = stage + tr_off[j] + ks * (TR_STEP_ROWS * TR_PITCH);
        const u32x2_t lo = lds_read_tr<ES>(p), hi = lds_read_tr<ES>(p + TR_HALF_ROWS * TR_PITCH);
        bf[set][j] = u32x4_t{lo[0], lo[1], hi[0], hi[1]};
      }
    }
  };
  auto mma = [&](int set) {
#pragma unroll
    for (int i = 0; i < FM; i++)
#pragma unroll
      for (int j = 0; j < FN; j++) acc[i][j] = mfma32<TYPES>(bf[set][j], af[set][i], acc[i][j]);
  };

  const int ktiles = K / BK;  // >= 1 on this path
  copy_slab(lds, 0);
  if (ktiles > 1) copy_slab(lds + STAGE_BYTES, BK);
  if (ktiles > 1) __builtin_amdgcn_s_waitcnt(0x0F70 | ((A_PW + B_PW) & 15) | (((A_PW + B_PW) >> 4) << 14));
  else __builtin_amdgcn_s_waitcnt(0x0F70);
  __syncthreads();
  read_frags(0, lds, 0);

  // One barrier per slab.  At the barrier of slab kt every wave has finished reading buffer kt&1 and the
  // copies of slab kt+1 have landed, so the copies of slab kt+2 may overwrite buffer kt&1 right after it;
  // they then have a whole slab of MFMAs to complete.
  if constexpr (F8) {
    auto mma2 = [&](int pair) {
#pragma unroll
      for (int i = 0; i < FM; i++)
#pragma unroll
        for (int j = 0; j < FN; j++)
          acc[i][j] = mfma_f8_pair<TYPES>(bf[2 * pair][j], bf[2 * pair + 1][j], af[2 * pair][i], af[2 * pair + 1][i], acc[i][j]);
    };
    read_frags(1, lds, 1);
    for (int kt = 0; kt < ktiles; kt++) {
      char* cur = lds + (kt & 1) * STAGE_BYTES;
      char* nxt = lds + ((kt + 1) & 1) * STAGE_BYTES;
      read_frags(2, cur, 2);
      read_frags(3, cur, 3);
      mma2(0);
      __builtin_amdgcn_sched_barrier(0);
      __builtin_amdgcn_s_waitcnt(0x0070);  // vmcnt(0) lgkmcnt(0)
      __syncthreads();
      if (kt + 2 < ktiles) copy_slab(cur, (kt + 2) * BK);
      if (kt + 1 < ktiles) {
        read_frags(0, nxt, 0);
        read_frags(1, nxt, 1);
      }
      mma2(1);
      __builtin_amdgcn_sched_barrier(0);
    }
  } else
  for (int kt = 0; kt < ktiles; kt++) {
    char* cur = lds + (kt & 1) * STAGE_BYTES;
    char* nxt = lds + ((kt + 1) & 1) * STAGE_BYTES;
#pragma unroll
    for (int ks = 0; ks < KSTEPS - 1; ks++) {
      read_frags((ks + 1) & 1, cur, ks + 1);
      mma(ks & 1);
      __builtin_amdgcn_sched_barrier(0);
    }
    __builtin_amdgcn_s_waitcnt(0x0070);  // vmcnt(0) lgkmcnt(0): my copies landed, my fragment reads returned
    __syncthreads();
    if (kt + 2 < ktiles) copy_slab(cur, (kt + 2) * BK);
    if (kt + 1 < ktiles) read_frags(KSTEPS & 1, nxt, 0);
    mma((KSTEPS - 1) & 1);
    __builtin_amdgcn_sched_barrier(0);
  }

  static_assert(NW * epilogue_region_bytes<FN>() <= 2 * STAGE_BYTES, "the epilogue reuses the operand buffers");
  __builtin_amdgcn_s_waitcnt(0x0070);  // no copy of this wave is still on its way into LDS
  __syncthreads();
  store_accumulators_lds<TYPES, FM, FN>(g, acc, m0 + wm * WM, n0 + wn * WN, lane, lds + wave * epilogue_region_bytes<FN>());
}

// ---------------------------------------------------------------------------
// Pieces of the hand-scheduled kernel (rung4_mfma_ring16.hpp).  Its main loop is a fixed instruction sequence
// written as volatile asm statements, so that neither the scheduler nor the wait-count pass (which, with an LDS copy
// pending, waits for lgkmcnt(0) before the first MFMA of every step) can change it; every s_waitcnt is placed by hand.
// ---------------------------------------------------------------------------
template <int OFF> __device__ __forceinline__ void asm_ds_read16(u32x4_t& dst, uint32_t addr) {
  asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "i"(OFF));
}
// LDS destination base of the following copies.  Writing M0 waits for the copies already queued to read it,
// which can hold up the wave's whole instruction stream, so it is written once per group of copies; the copies
// of a group step through LDS with their immediate offset.
__device__ __forceinline__ void asm_set_m0(uint32_t lds_addr) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0" : : "s"(lds_addr) : "memory");
}
// 64 lanes x 16 bytes from sbase + voff + OFF (per lane) to LDS at M0 + OFF + 16 * lane: the immediate offset
// applies to both addresses, so the caller takes OFF off the source address again (in sbase or in voff).
template <int OFF> __device__ __forceinline__ void asm_copy16(uint32_t voff, const void* sbase) {
  static_assert(OFF >= -4096 && OFF <= 4095, "13-bit signed immediate");
  asm volatile("global_load_lds_dwordx4 %0, %1 offset:%2" : : "v"(voff), "s"(sbase), "i"(OFF) : "memory");
}
typedef uint32_t u32x8_t __attribute__((ext_vector_type(8)));
// half a fragment of a row-major B through the transposing LDS reads
template <int ES, int OFF> __device__ __forceinline__ void asm_ds_read_tr(u32x2_t& dst, uint32_t addr) {
  if constexpr (ES == 2) asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "i"(OFF));
  else asm volatile("ds_read_b64_tr_b8 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "i"(OFF));
}

}  // namespace gz

#include "rung4_mfma_ring16.hpp"

namespace gz {

// ---------------------------------------------------------------------------
// Launcher
// ---------------------------------------------------------------------------
template <int TYPES, int BM, int BN, int WAVES_M, int WAVES_N>
static int launch_cfg(const GemmArgs<TYPES>& g, int shape_class, int ring, hipStream_t s, bool transposed = false) {
  const int tiles_m = ceil_div(g.M, BM), tiles_n = ceil_div(g.N, BN);
  const dim3 grid((unsigned)(tiles_m * tiles_n)), block(WAVES_M * WAVES_N * 64);
  const size_t lds = 2u * (size_t)(BM + BN) * PITCH;
  const bool akc = g.layoutA == GZ_ROW_MAJOR, bkc = g.layoutB == GZ_COL_MAJOR;

#define GZ_LAUNCH(AKC, BKC, EDGE)                                                                   \
  do {                                                                                              \
    auto kern = mfma_gemm_kernel<TYPES, BM, BN, WAVES_M, WAVES_N, AKC, BKC, EDGE>;                   \
    GZ_SET_LDS_LIMIT(kern, lds);                                                                    \
    hipLaunchKernelGGL(kern, grid, block, lds, s, g, tiles_m, tiles_n);                             \
  } while (0)

  const bool edge = shape_class != MFMA_SHAPE_WHOLE;
  // one launch of a direct-to-LDS kernel and out
#define GZ_LAUNCH_DIRECT_ON(GRID, KERN, LDS_BYTES, ...)                                             \
  do {                                                                                              \
    auto kern = KERN;                                                                               \
    GZ_SET_LDS_LIMIT(kern, LDS_BYTES);                                                              \
    hipLaunchKernelGGL(kern, GRID, block, LDS_BYTES, s, g, tiles_m, tiles_n, ##__VA_ARGS__);        \
    GZ_HIP_TRY(hipGetLastError());                                                                  \
    return GZ_OK;                                                                                   \
  } while (0)
#define GZ_LAUNCH_DIRECT(KERN, LDS_BYTES, ...) GZ_LAUNCH_DIRECT_ON(grid, GZ_KERN(KERN), LDS_BYTES, ##__VA_ARGS__)
#define GZ_KERN(...) __VA_ARGS__   // a template-id with commas as one macro argument

  // The direct-to-LDS kernels: row-major A, whole K slabs, 16-byte aligned rows (the shape class says so), whole
  // tiles or, on the hand-scheduled 256 x 256 kernel, any M and N (rows clamped).  ring: 0 the compiler-scheduled
  // kernels, 1 the hand-scheduled ring kernel with one work-group per compute unit walking the tiles of a grid of
  // more than one round (ragged M and N included), 2 the same kernel with one work-group per tile.
  constexpr bool TILE_256 = BM == 256 && BN == 256 && WAVES_M == 2 && (WAVES_N == 2 || WAVES_N == 4);
  const size_t ring_lds = 5u * (size_t)(BM + BN) * 64;
  const size_t dtl_lds = 2u * (size_t)(BM + BN) * SLAB_BYTES;
  const dim3 pgrid((unsigned)(ring == 1 ? mfma_persistent_grid((long long)tiles_m * tiles_n, device_compute_units())
                                        : (long long)tiles_m * tiles_n));
  // fp32 on the hand-scheduled kernel: the 256 x 256 tile on four waves, a row-major A with either layout of B, and
  // two column-major operands as the transposed problem (v_mfma_f32_16x16x4_f32, four per block and K step)
  if constexpr (TYPES == GZ_F32F32F32 && TILE_256 && WAVES_N == 2) {
    if (transposed) {
      if (ring && shape_class == MFMA_SHAPE_RAGGED_MN)
        GZ_LAUNCH_DIRECT_ON(pgrid, GZ_KERN(mfma_ring16_kernel<TYPES, BM, BN, WAVES_N, WAVES_M, true, false, false, true>), ring_lds, StreamK{});
      if (ring && !edge)
        GZ_LAUNCH_DIRECT_ON(pgrid, GZ_KERN(mfma_ring16_kernel<TYPES, BM, BN, WAVES_N, WAVES_M, false, false, false, true>), ring_lds, StreamK{});
      set_error("mfma rung: no kernel for the transposed problem on this tile");
      return GZ_ERR_UNSUPPORTED;
    }
    if (ring && akc && shape_class == MFMA_SHAPE_RAGGED_MN) {
      if (bkc) GZ_LAUNCH_DIRECT_ON(pgrid, GZ_KERN(mfma_ring16_kernel<TYPES, BM, BN, WAVES_M, WAVES_N, true>), ring_lds, StreamK{});
      else GZ_LAUNCH_DIRECT_ON(pgrid, GZ_KERN(mfma_ring16_kernel<TYPES, BM, BN, WAVES_M, WAVES_N, true, false, false>), ring_lds, StreamK{});
    }
    if (ring && akc && !edge) {
      if (bkc) GZ_LAUNCH_DIRECT_ON(pgrid, GZ_KERN(mfma_ring16_kernel<TYPES, BM, BN, WAVES_M, WAVES_N>), ring_lds, StreamK{});
      else GZ_LAUNCH_DIRECT_ON(pgrid, GZ_KERN(mfma_ring16_kernel<TYPES, BM, BN, WAVES_M, WAVES_N, false, false, false>), ring_lds, StreamK{});
    }
  }
  // (and the 128 x 128 tile of the same kernel on whole tiles, two work-groups per compute unit)
  if constexpr (TYPES == GZ_F32F32F32 && BM == 128 && BN == 128 && WAVES_M == 2 && WAVES_N == 2) {
    if (transposed) {
      if (ring && !edge)
        GZ_LAUNCH_DIRECT(GZ_KERN(mfma_ring16_kernel<TYPES, BM, BN, WAVES_N, WAVES_M, false, false, false, true>), ring_lds, StreamK{});
      set_error("mfma rung: no kernel for the transposed problem on this tile");
      return GZ_ERR_UNSUPPORTED;
    }
    if (ring && akc && !edge) {
      if (bkc) GZ_LAUNCH_DIRECT(GZ_KERN(mfma_ring16_kernel<TYPES, BM, BN, WAVES_M, WAVES_N>), ring_lds, StreamK{});
      else GZ_LAUNCH_DIRECT(GZ_KERN(mfma_ring16_kernel<TYPES, BM, BN, WAVES_M, WAVES_N, false, false, false>), ring_lds, StreamK{});
    }
  }
  if constexpr (TYPES != GZ_F32F32F32) {
    // `transposed`: g is the transposed problem of a column-major A with a column-major B (see SWAP in
    // rung4_mfma_ring16.hpp), a row-major pair for the ring kernel's operands, with the real C and D
    // (the waves of a tile laid out the other way round as well: the wave count along the real M stays what it is)
    if (transposed) {
      if constexpr (TILE_256 && !(is_fp8(TYPES) && WAVES_M * WAVES_N == 8)) {
        if (ring && shape_class == MFMA_SHAPE_RAGGED_MN)
          GZ_LAUNCH_DIRECT_ON(pgrid, GZ_KERN(mfma_ring16_kernel<TYPES, BM, BN, WAVES_N, WAVES_M, true, false, false, true>), ring_lds, StreamK{});
        if (ring && !edge)
          GZ_LAUNCH_DIRECT_ON(pgrid, GZ_KERN(mfma_ring16_kernel<TYPES, BM, BN, WAVES_N, WAVES_M, false, false, false, true>), ring_lds, StreamK{});
      }
      if constexpr (BM == 128 && BN == 128 && WAVES_M == 2 && WAVES_N == 2 && !is_fp8(TYPES)) {
        if (ring && !edge)
          GZ_LAUNCH_DIRECT(GZ_KERN(mfma_ring16_kernel<TYPES, BM, BN, WAVES_N, WAVES_M, false, false, false, true>), ring_lds, StreamK{});
      }
      set_error("mfma rung: no kernel for the transposed problem on this tile");
      return GZ_ERR_UNSUPPORTED;
    }
    // a column-major A with a row-major B (int8 and the 16-bit types): both operands through the transposing reads
    if constexpr (!is_fp8(TYPES)) {
      if constexpr (TILE_256) {
        if (ring && !akc && !bkc && shape_class == MFMA_SHAPE_RAGGED_MN)
          GZ_LAUNCH_DIRECT_ON(pgrid, GZ_KERN(mfma_ring16_kernel<TYPES, BM, BN, WAVES_M, WAVES_N, true, false, false, false, false>), ring_lds, StreamK{});
        if (ring && !akc && !bkc && !edge)
          GZ_LAUNCH_DIRECT_ON(pgrid, GZ_KERN(mfma_ring16_kernel<TYPES, BM, BN, WAVES_M, WAVES_N, false, false, false, false, false>), ring_lds, StreamK{});
      }
      if constexpr (BM == 128 && BN == 128 && WAVES_M == 2 && WAVES_N == 2) {
        if (ring && !akc && !bkc && !edge)
          GZ_LAUNCH_DIRECT(GZ_KERN(mfma_ring16_kernel<TYPES, BM, BN, WAVES_M, WAVES_N, false, false, false, false, false>), ring_lds, StreamK{});
      }
    }
    if constexpr (TILE_256) {
      if (ring && akc && shape_class == MFMA_SHAPE_RAGGED_MN) {
        if (bkc) GZ_LAUNCH_DIRECT_ON(pgrid, GZ_KERN(mfma_ring16_kernel<TYPES, BM, BN, WAVES_M, WAVES_N, true>), ring_lds, StreamK{});
        else GZ_LAUNCH_DIRECT_ON(pgrid, GZ_KERN(mfma_ring16_kernel<TYPES, BM, BN, WAVES_M, WAVES_N, true, false, false>), ring_lds, StreamK{});
      }
      if (ring && akc && !edge) {
        if (bkc) GZ_LAUNCH_DIRECT_ON(pgrid, GZ_KERN(mfma_ring16_kernel<TYPES, BM, BN, WAVES_M, WAVES_N>), ring_lds, StreamK{});
        else GZ_LAUNCH_DIRECT_ON(pgrid, GZ_KERN(mfma_ring16_kernel<TYPES, BM, BN, WAVES_M, WAVES_N, false, false, false>), ring_lds, StreamK{});
      }
    }
    // the same kernel on whole 128 x 128 tiles (int8 and the 16-bit types), one work-group per tile, two per compute unit
    if constexpr (BM == 128 && BN == 128 && WAVES_M == 2 && WAVES_N == 2 && !is_fp8(TYPES)) {
      if (ring && akc && !edge) {
        if (bkc) GZ_LAUNCH_DIRECT(GZ_KERN(mfma_ring16_kernel<TYPES, BM, BN, WAVES_M, WAVES_N>), ring_lds, StreamK{});
        else GZ_LAUNCH_DIRECT(GZ_KERN(mfma_ring16_kernel<TYPES, BM, BN, WAVES_M, WAVES_N, false, false, false>), ring_lds, StreamK{});
      }
    }
    if (!edge && akc && bkc) {  // whole tiles, both operands K-contiguous
      // The compiler-scheduled direct-to-LDS kernel is kept for the eight-wave 256x256 tile only: with four waves the
      // register-staged kernel below, whose loads and LDS stores are spread between the MFMAs, measured faster on
      // every tile (interleaved runs, us, direct / register-staged: bf16 2048^3 128x128 28.6 / 27.1, 256x128 39.2 /
      // 37.0; 4096^3 256x256 130.1 / 121.9; int8 8192^3 512 / 495; fp8 8192^3 479 / 424).
      if constexpr (WAVES_M * WAVES_N == 8) GZ_LAUNCH_DIRECT(GZ_KERN(mfma_dtl_kernel<TYPES, BM, BN, WAVES_M, WAVES_N>), dtl_lds);
    }
    if (!edge && akc && !bkc) {  // whole tiles, row-major A and B: direct-to-LDS copies, transposing LDS reads for B
      // (128x128 only: on 256x128 the register-staged kernel is faster, 2048^3 50.0 / 43.0 us, 4096^3 185 / 150)
      if constexpr (BM == 128 && BN == 128) GZ_LAUNCH_DIRECT(GZ_KERN(mfma_dtl_kernel<TYPES, BM, BN, WAVES_M, WAVES_N, false>), dtl_lds);
    }
  }
#undef GZ_LAUNCH_DIRECT
#undef GZ_LAUNCH_DIRECT_ON
#undef GZ_KERN
  if (edge) {
    if (akc && bkc) GZ_LAUNCH(true, true, true);
    else if (akc && !bkc) GZ_LAUNCH(true, false, true);
    else if (!akc && bkc) GZ_LAUNCH(false, true, true);
    else GZ_LAUNCH(false, false, true);
  } else {
    if (akc && bkc) GZ_LAUNCH(true, true, false);
    else if (akc && !bkc) GZ_LAUNCH(true, false, false);
    else if (!akc && bkc) GZ_LAUNCH(false, true, false);
    else GZ_LAUNCH(false, false, false);
  }
#undef GZ_LAUNCH
  GZ_HIP_TRY(hipGetLastError());
  return GZ_OK;
}

// ---------------------------------------------------------------------------
// The last few columns of a problem whose N is just past a multiple of 256 (see mfma_resolve_colsplit), at most
// STRIP_MAX_COLS of them: g.N columns, g.B / g.C / g.D pointing at the first of them, ldb / ldd the pitch of the
// whole matrices.  As a tile problem this strip is all edge (fp16 4095 x 1 x 1023 took 47 us on 128 x 128 tiles, most
// of it element-wise loads of one column of B); as M dot products per column it is one pass over A.  One wave per
// row, four rows per wave: the lanes take 16-byte pieces of the row and of the columns (staged in LDS), multiply-add on
// the vector ALUs in the accumulator type, and meet in a butterfly over the 64 lanes.
// ---------------------------------------------------------------------------
constexpr int STRIP_WAVES = 4, STRIP_ROWS_PER_WAVE = 4, STRIP_ROWS_PER_WG = STRIP_WAVES * STRIP_ROWS_PER_WAVE;
template <int TYPES, bool A_KC, bool B_KC, int R>
__global__ void __launch_bounds__(STRIP_WAVES * 64) mfma_strip_kernel(GemmArgs<TYPES> g) {
  using T = Traits<TYPES>;
  using in_t = typename T::in_t;
  using acc_t = typename T::acc_t;
  constexpr int EPV = 16 / (int)sizeof(in_t);
  // The columns of B go through LDS, K-contiguous, once per work-group: gathered by every wave from a row-major B
  // (one cache line per element) they were most of the kernel's time (19 us for one column of 1023).
  // A chunk of K is 4 x 64 lanes x 16 bytes, whatever the element size: per chunk a lane holds four 16-byte pieces
  // of each of its wave's rows, and all of those loads and the gather of B are issued before anything waits for
  // them (row by row and piece by piece, each behind its own wait, fp16 4095 x 1 x 1023 took 10.8 us).
  constexpr int KI = 4, K_CHUNK = KI * 64 * EPV, GI = K_CHUNK / (STRIP_WAVES * 64);
  __shared__ __attribute__((aligned(16))) in_t bs[R * K_CHUNK];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int m0 = blockIdx.x * STRIP_ROWS_PER_WG + wave * STRIP_ROWS_PER_WAVE;
  const int K = g.K, M = g.M, r = g.N;
  const size_t lda = (size_t)g.lda, ldb = (size_t)g.ldb;
  acc_t acc[STRIP_ROWS_PER_WAVE][R];
#pragma unroll
  for (int i = 0; i < STRIP_ROWS_PER_WAVE; i++)
#pragma unroll
    for (int j = 0; j < R; j++) acc[i][j] = 0;
  // element e of a 16-byte piece held as four words, and an element's bits as a word
  constexpr int EBITS = 8 * (int)sizeof(in_t), EPW = 4 / (int)sizeof(in_t);
  auto elem_bits = [](in_t x) -> uint32_t {
    if constexpr (sizeof(in_t) == 1) return (uint32_t)__builtin_bit_cast(uint8_t, x);
    else if constexpr (sizeof(in_t) == 2) return (uint32_t)__builtin_bit_cast(uint16_t, x);
    else return __builtin_bit_cast(uint32_t, x);
  };
  auto elem_of = [](const u32x4_t& v, int e) -> in_t {
    const uint32_t w = v[e / EPW] >> (e % EPW * EBITS);
    if constexpr (sizeof(in_t) == 1) return __builtin_bit_cast(in_t, (uint8_t)w);
    else if constexpr (sizeof(in_t) == 2) return __builtin_bit_cast(in_t, (uint16_t)w);
    else return __builtin_bit_cast(in_t, w);
  };
  // element e widened to the accumulator's type (the 8-bit floats by the conversion instruction, which takes the
  // word and a byte number)
  auto widen_elem = [&](const u32x4_t& v, int e) -> acc_t {
    if constexpr (TYPES == GZ_E4M3E4M3F16 || TYPES == GZ_E5M2E5M2F16) {
      const int w = (int)v[e / 4];
#define GZ_CVT(SEL) (TYPES == GZ_E4M3E4M3F16 ? __builtin_amdgcn_cvt_f32_fp8(w, SEL) : __builtin_amdgcn_cvt_f32_bf8(w, SEL))
      switch (e % 4) {   // (the byte number is part of the instruction; e is a constant once the loops are unrolled)
        case 0: return GZ_CVT(0);
        case 1: return GZ_CVT(1);
        case 2: return GZ_CVT(2);
        default: return GZ_CVT(3);
      }
#undef GZ_CVT
    } else {
      return widen_in<TYPES>(elem_of(v, e));
    }
  };
  auto mac = [&](acc_t a, acc_t b, acc_t c) -> acc_t {
    if constexpr (T::is_int) return c + a * b;
    else return __builtin_fmaf(a, b, c);
  };
  // the elements of a row of A that the 16-byte pieces cover
  const int k_vec_end = A_KC ? K / EPV * EPV : K;
  for (int kc0 = 0; kc0 < K; kc0 += K_CHUNK) {
    const int kn = min(K_CHUNK, K - kc0), kn_pad = (kn + EPV - 1) / EPV * EPV;   // zero-filled up to whole vectors
    // This lane's pieces of its wave's rows.  Every load is unconditional, from an address clamped into the matrix,
    // and what lies past the end is zeroed where it is used: a load under a lane-dependent condition ends in a merge
    // that waits for it, one load at a time.  A K-contiguous A is read in whole 16-byte pieces only (a lane whose
    // piece would reach past the last whole one reads that one instead); the K % EPV elements after them are added
    // at the end.  A step of the wave that lies past the end altogether is skipped (the same for all lanes).
    // (pieces are kept as four 32-bit words and taken apart by shifts: an array of bytes that is written both as a
    // whole and element by element stays in scratch memory)
    u32x4_t a[STRIP_ROWS_PER_WAVE][KI];
#pragma unroll
    for (int i = 0; i < STRIP_ROWS_PER_WAVE; i++)
#pragma unroll
      for (int t = 0; t < KI; t++) {
        const int m = min(m0 + i, M - 1), k = kc0 + (t * 64 + lane) * EPV;
        a[i][t] = u32x4_t{0, 0, 0, 0};
        if (kc0 + t * 64 * EPV >= k_vec_end) continue;
        if constexpr (A_KC) {
          __builtin_memcpy(&a[i][t], g.A + (size_t)m * lda + min(k, k_vec_end - EPV), 16);
        } else {
          u32x4_t v = {0, 0, 0, 0};
#pragma unroll
          for (int e = 0; e < EPV; e++) {
            const int kk = min(k + e, K - 1);
            v[e / EPW] |= elem_bits(g.A[(size_t)kk * lda + m]) << (e % EPW * EBITS);
          }
          a[i][t] = v;
        }
      }
    // the strip's columns of B into LDS
    for (int j = 0; j < r; j++) {
      in_t tmp[GI];
#pragma unroll
      for (int t = 0; t < GI; t++) {
        tmp[t] = (in_t)0;
        if (t * STRIP_WAVES * 64 >= kn) continue;   // (the same for all lanes)
        const int kk = min(kc0 + (int)threadIdx.x + t * STRIP_WAVES * 64, K - 1);
        tmp[t] = B_KC ? g.B[(size_t)j * ldb + kk] : g.B[(size_t)kk * ldb + j];
      }
#pragma unroll
      for (int t = 0; t < GI; t++) {
        const int k = (int)threadIdx.x + t * STRIP_WAVES * 64;
        if (k < kn_pad) bs[j * K_CHUNK + k] = k < kn ? tmp[t] : (in_t)0;
      }
    }
    __syncthreads();
    // (pieces and columns are unrolled by construction: an unroll request for a body this large is declined for the
    // 8-bit types, and the pieces, indexed by a loop counter, then live in scratch memory.)  Per piece the elements
    // of the rows are widened once, those of a column once, and each sum takes its products in ascending k.  Rows
    // past M hold row M - 1 again and are never written.
    static_for<KI>([&](auto t_c) {
      constexpr int t = decltype(t_c)::value;
      const int k0 = (t * 64 + lane) * EPV;
      if (k0 < kn_pad) {
        acc_t aw[STRIP_ROWS_PER_WAVE][EPV];
#pragma unroll
        for (int i = 0; i < STRIP_ROWS_PER_WAVE; i++)
#pragma unroll
          for (int e = 0; e < EPV; e++)   // b is zero past the end of K; a may be anything there (a NaN of the next row)
            aw[i][e] = kc0 + k0 + e < k_vec_end ? widen_elem(a[i][t], e) : (acc_t)0;
        static_for<R>([&](auto j_c) {
          constexpr int j = decltype(j_c)::value;
          if (j < r) {   // the same for every lane
            const u32x4_t b = *reinterpret_cast<const u32x4_t*>(bs + j * K_CHUNK + k0);
#pragma unroll
            for (int e = 0; e < EPV; e++) {
              const acc_t bw = widen_elem(b, e);
#pragma unroll
              for (int i = 0; i < STRIP_ROWS_PER_WAVE; i++) acc[i][j] = mac(aw[i][e], bw, acc[i][j]);
            }
          }
        });
      }
    });
    __syncthreads();
  }
  // the last K % EPV elements of the rows of a K-contiguous A, one per lane
  if constexpr (A_KC) {
    if (k_vec_end < K) {
      const int kk = min(k_vec_end + lane, K - 1);
      const bool mine = k_vec_end + lane < K;
      static_for<R>([&](auto j_c) {
        constexpr int j = decltype(j_c)::value;
        if (j < r) {
          const in_t bv = B_KC ? g.B[(size_t)j * ldb + kk] : g.B[(size_t)kk * ldb + j];
          const acc_t bw = mine ? widen_in<TYPES>(bv) : (acc_t)0;
#pragma unroll
          for (int i = 0; i < STRIP_ROWS_PER_WAVE; i++) {
            const in_t av = g.A[(size_t)min(m0 + i, M - 1) * lda + kk];
            acc[i][j] = mac(mine ? widen_in<TYPES>(av) : (acc_t)0, bw, acc[i][j]);
          }
        }
      });
    }
  }
#pragma unroll
  for (int i = 0; i < STRIP_ROWS_PER_WAVE; i++) {
    const int m = m0 + i;
    if (m >= M) break;
#pragma unroll
    for (int j = 0; j < R; j++) {
      acc_t v = acc[i][j];
#pragma unroll
      for (int off = 32; off >= 1; off >>= 1) v += __shfl_xor(v, off, 64);
      if (lane == 0 && j < r) {
        g.D[(size_t)m * g.ldd + j] = epilogue<TYPES>(v, g.alpha, g.beta, g.C + (size_t)m * g.ldc + j);
      }
    }
  }
}

template <int TYPES> static int launch_strip(const GemmArgs<TYPES>& g, hipStream_t s) {
  const dim3 grid((unsigned)ceil_div(g.M, STRIP_ROWS_PER_WG)), block(STRIP_WAVES * 64);
  const bool akc = g.layoutA == GZ_ROW_MAJOR, bkc = g.layoutB == GZ_COL_MAJOR;
#define GZ_STRIP(AKC, BKC)                                                                              \
  do {                                                                                                  \
    if (g.N <= 1) hipLaunchKernelGGL((mfma_strip_kernel<TYPES, AKC, BKC, 1>), grid, block, 0, s, g);     \
    else if (g.N <= 4) hipLaunchKernelGGL((mfma_strip_kernel<TYPES, AKC, BKC, 4>), grid, block, 0, s, g); \
    else hipLaunchKernelGGL((mfma_strip_kernel<TYPES, AKC, BKC, MFMA_STRIP_MAX_COLS>), grid, block, 0, s, g); \
  } while (0)
  if (akc && bkc) GZ_STRIP(true, true);
  else if (akc) GZ_STRIP(true, false);
  else if (bkc) GZ_STRIP(false, true);
  else GZ_STRIP(false, false);
#undef GZ_STRIP
  GZ_HIP_TRY(hipGetLastError());
  return GZ_OK;
}

template <int TYPES> static int launch_one(const GemmArgs<TYPES>& g, const MfmaCfg& chosen, hipStream_t s, bool adjust = false,
                                           bool transposed = false) {
  using in_t = typename Traits<TYPES>::in_t;
  MfmaCfg cfg = chosen;
  const int edge = mfma_launch_class(cfg, (int)sizeof(in_t), (int)sizeof(typename Traits<TYPES>::out_t), g.M, g.N, g.K,
                                     g.layoutA, g.layoutB, g.A, g.B, g.C, g.D, g.lda, g.ldb, g.ldc, g.ldd);
  if (adjust) mfma_adjust_general(TYPES, edge, g.layoutA, g.layoutB, &cfg);   // launcher's choice: the wave count follows the kernel
  switch (cfg.id) {
    case 1: return launch_cfg<TYPES, 256, 256, 2, 2>(g, edge, 0, s);
    case 2: return launch_cfg<TYPES, 256, 256, 2, 4>(g, edge, 0, s);
    case 3: return launch_cfg<TYPES, 128, 128, 2, 2>(g, edge, 0, s);
    case 4: return launch_cfg<TYPES, 256, 128, 2, 2>(g, edge, 0, s);
    case 5: case 7: return launch_cfg<TYPES, 256, 256, 2, 2>(g, edge, 1, s, transposed);
    case 6: case 8: return launch_cfg<TYPES, 256, 256, 2, 4>(g, edge, 1, s, transposed);
    case 9: return launch_cfg<TYPES, 256, 256, 2, 2>(g, edge, 2, s, transposed);
    case 10: return launch_cfg<TYPES, 256, 256, 2, 4>(g, edge, 2, s, transposed);
    case 11: return launch_cfg<TYPES, 128, 128, 2, 2>(g, edge, 2, s, transposed);
    case 12:   // (8-bit elements on two waves)
      if constexpr (sizeof(in_t) >= 2) return launch_cfg<TYPES, 64, 64, 2, 2>(g, edge, 0, s);
      else return launch_cfg<TYPES, 64, 64, 1, 2>(g, edge, 0, s);
    default: break;
  }
  set_error("mfma rung: variant %d not built", cfg.id);
  return GZ_ERR_UNSUPPORTED;
}

// Stream-K: the whole tiles and the runs of the remaining tiles' slabs in one launch, then the launch that adds the
// pieces (see struct StreamK).  The workspace comes from workspace_acquire: the library's own pool, or the static
// buffer of the entry point that allocates nothing.
template <int TYPES, int WAVES_N>
static int launch_streamk(const GemmArgs<TYPES>& g, const StreamKPlan& p, bool ragged, hipStream_t s) {
  if constexpr (is_fp8(TYPES) || TYPES == GZ_F32F32F32 || is_acc16(TYPES)) {
    set_error("mfma rung: no stream-K kernel for this type bundle");
    return GZ_ERR_UNSUPPORTED;
  } else {
    void* ws = nullptr;
    const int st = workspace_acquire((size_t)p.slots * MFMA_STREAMK_SLOT_BYTES, s, &ws);
    if (st != GZ_OK) return st;
    StreamK sk{p.dp_tiles, p.sk_tiles, p.blocks, p.q, p.rem, ws};
    const int tiles_m = ceil_div(g.M, 256), tiles_n = ceil_div(g.N, 256);
    const dim3 grid((unsigned)(p.dp_tiles + p.blocks)), block(2 * WAVES_N * 64);
    const size_t rlds = 5u * (size_t)(256 + 256) * 64;
#define GZ_LAUNCH_SK(RAGGED_, BKC_)                                                    \
  do {                                                                                 \
    auto kern = mfma_ring16_kernel<TYPES, 256, 256, 2, WAVES_N, RAGGED_, true, BKC_>;  \
    GZ_SET_LDS_LIMIT(kern, rlds);                                                      \
    hipLaunchKernelGGL(kern, grid, block, rlds, s, g, tiles_m, tiles_n, sk);           \
  } while (0)
    const bool bkc = g.layoutB == GZ_COL_MAJOR;
    if (ragged && bkc) GZ_LAUNCH_SK(true, true);
    else if (ragged) GZ_LAUNCH_SK(true, false);
    else if (bkc) GZ_LAUNCH_SK(false, true);
    else GZ_LAUNCH_SK(false, false);
#undef GZ_LAUNCH_SK
    GZ_HIP_TRY(hipGetLastError());
    hipLaunchKernelGGL((streamk_fixup_kernel<TYPES>), dim3((unsigned)p.sk_tiles * 64), dim3(256), 0, s, g, tiles_m, tiles_n, sk);
    GZ_HIP_TRY(hipGetLastError());
    return GZ_OK;
  }
}

template <int TYPES> int launch_mfma(const GemmArgs<TYPES>& args, int variant, hipStream_t s) {
  GemmArgs<TYPES> g = args;
  const int num_cus = device_compute_units();
  g.store_hint = mfma_store_hint(TYPES, g.M, g.N, g.K, (int)sizeof(typename Traits<TYPES>::out_t), num_cus);
  // Column-major A and B: the transposed problem on the ring kernel - one launch, or where the launcher would cut
  // the rows of the transposed problem (a mostly empty last round) two, over column ranges of the real C and D.
  // Returns -1 where that kernel does not take the problem.
  auto run_transposed = [&](const GemmArgs<TYPES>& gm, bool allow_split) -> int {
    MfmaSplit tsp;
    MfmaCfg ct;
    if (!mfma_transposed_ring(TYPES, gm.M, gm.N, gm.K, gm.layoutA, gm.layoutB, variant, num_cus, &ct, allow_split ? &tsp : nullptr))
      return -1;
    if (!allow_split) tsp.rows_main = 0;
    GemmArgs<TYPES> t = gm;
    t.A = gm.B; t.B = gm.A;
    t.M = gm.N; t.N = gm.M;
    t.lda = gm.ldb; t.ldb = gm.lda;
    t.layoutA = GZ_ROW_MAJOR; t.layoutB = GZ_ROW_MAJOR;
    auto cls_of = [&](const GemmArgs<TYPES>& a, const MfmaCfg& c) {
      return mfma_launch_class(c, (int)sizeof(typename Traits<TYPES>::in_t), (int)sizeof(typename Traits<TYPES>::out_t), a.M, a.N,
                               a.K, a.layoutA, a.layoutB, a.A, a.B, a.C, a.D, a.lda, a.ldb, a.ldc, a.ldd);
    };
    if (tsp.rows_main > 0) {
      GemmArgs<TYPES> top = t, bottom = t;
      top.M = tsp.rows_main;
      bottom.M = t.M - tsp.rows_main;
      bottom.A = t.A + (size_t)tsp.rows_main * (size_t)t.lda;   // rows of the transposed problem: columns of B, C and D
      if (t.C) bottom.C = t.C + tsp.rows_main;
      bottom.D = t.D + tsp.rows_main;
      if (cls_of(top, tsp.main) == MFMA_SHAPE_WHOLE && cls_of(bottom, tsp.tail) == MFMA_SHAPE_WHOLE) {
        const int st = launch_one<TYPES>(top, tsp.main, s, false, true);
        if (st != GZ_OK) return st;
        return launch_one<TYPES>(bottom, tsp.tail, s, false, true);
      }
      (void)mfma_choose(TYPES, t.M, t.N, t.K, t.layoutA, t.layoutB, num_cus, &ct);   // odd pitches: one launch
      if (ct.ring == 0) ct = kMfmaCfgs[MFMA_CFG_RING_W4];
    }
    const int cls = cls_of(t, ct);
    // (unaligned operands, or rows of D that are not: the kernels of the problem as given, below)
    if (cls == MFMA_SHAPE_WHOLE || (cls == MFMA_SHAPE_RAGGED_MN && ct.bm == 256)) return launch_one<TYPES>(t, ct, s, false, true);
    return -1;
  };
  // (a few columns past a multiple of 256 are cut off first, as for the other layouts: the transposed problem would
  // carry them as a whole row of tiles - bf16 4096 x 4104 x 4096 170 us in one launch)
  MfmaColSplit ccs;
  if (variant == 0 && g.K > 0 && g.layoutA == GZ_COL_MAJOR && g.layoutB == GZ_COL_MAJOR &&
      mfma_resolve_colsplit(TYPES, g.M, g.N, g.K, g.layoutA, g.layoutB, num_cus, &ccs)) {
    GemmArgs<TYPES> left = g, right = g;
    left.N = ccs.cols_main;
    right.N = g.N - ccs.cols_main;
    right.B = g.B + (size_t)ccs.cols_main * (size_t)g.ldb;
    if (g.C) right.C = g.C + ccs.cols_main;
    right.D = g.D + ccs.cols_main;
    const int st = run_transposed(left, false);
    if (st > 0) return st;
    if (st == GZ_OK) return ccs.strip ? launch_strip<TYPES>(right, s) : launch_one<TYPES>(right, ccs.tail, s, true);
  } else if (const int st = run_transposed(g, true); st >= 0) {
    return st;
  }
  if ((variant == 0 || variant == MFMA_VARIANT_STREAMK_W4 || variant == MFMA_VARIANT_STREAMK_W8) && g.K > 0) {
    StreamKPlan skp;
    const MfmaCfg* forced = variant == 0 ? nullptr : &kMfmaCfgs[variant - 1];
    // the launcher's own choice stays within the workspace this entry point may use (the entry point that
    // allocates nothing has a fixed one); an explicit stream-K variant is refused by workspace_acquire instead
    if (mfma_plan_streamk(TYPES, g.M, g.N, g.K, g.layoutA, g.layoutB, num_cus, forced != nullptr, forced, &skp) &&
        (forced || (size_t)skp.slots * MFMA_STREAMK_SLOT_BYTES <= workspace_limit())) {
      const int cls = mfma_launch_class(skp.cfg, (int)sizeof(typename Traits<TYPES>::in_t),
                                        (int)sizeof(typename Traits<TYPES>::out_t), g.M, g.N, g.K, g.layoutA, g.layoutB,
                                        g.A, g.B, g.C, g.D, g.lda, g.ldb, g.ldc, g.ldd);
      if (cls != MFMA_SHAPE_GENERAL) {   // (unaligned operands: the plain launch below, on the register-staged kernel)
        g.store_hint = 0;   // one round at most ends in each launch: plain stores
        return skp.cfg.waves_n == 4 ? launch_streamk<TYPES, 4>(g, skp, cls == MFMA_SHAPE_RAGGED_MN, s)
                                    : launch_streamk<TYPES, 2>(g, skp, cls == MFMA_SHAPE_RAGGED_MN, s);
      }
    }
  }
  if (variant == 0 && g.K > 0) {
    MfmaSplit sp;
    MfmaColSplit cs;
    const int cut = mfma_resolve_cut(TYPES, g.M, g.N, g.K, g.layoutA, g.layoutB, num_cus, &sp, &cs);
    if (cut == 1) {
      // a mostly empty last round of 256x256 tiles: the rows that fill whole rounds first, the rest in a second launch
      GemmArgs<TYPES> top = g, bottom = g;
      top.M = sp.rows_main;
      bottom.M = g.M - sp.rows_main;
      bottom.A = g.A + (size_t)sp.rows_main * (size_t)g.lda;   // row-major A: a row range is a matrix with the same pitch
      if (g.C) bottom.C = g.C + (size_t)sp.rows_main * (size_t)g.ldc;
      bottom.D = g.D + (size_t)sp.rows_main * (size_t)g.ldd;
      const int st = launch_one<TYPES>(top, sp.main, s, true);
      if (st != GZ_OK) return st;
      return launch_one<TYPES>(bottom, sp.tail, s, true);
    }
    if (cut == 2) {
      // a few columns past a multiple of 256: those columns in a launch of their own
      GemmArgs<TYPES> left = g, right = g;
      left.N = cs.cols_main;
      right.N = g.N - cs.cols_main;
      right.B = g.layoutB == GZ_ROW_MAJOR ? g.B + cs.cols_main : g.B + (size_t)cs.cols_main * (size_t)g.ldb;
      if (g.C) right.C = g.C + cs.cols_main;
      right.D = g.D + cs.cols_main;
      const int st = launch_one<TYPES>(left, cs.main, s, true);
      if (st != GZ_OK) return st;
      return cs.strip ? launch_strip<TYPES>(right, s) : launch_one<TYPES>(right, cs.tail, s, true);
    }
  }
  MfmaCfg cfg;
  if (!mfma_resolve(TYPES, g.M, g.N, g.K, g.layoutA, g.layoutB, variant, num_cus, &cfg)) {
    set_error("mfma rung: unknown variant %d", variant);
    return GZ_ERR_UNSUPPORTED;
  }
  return launch_one<TYPES>(g, cfg, s, variant == 0);
}

}  // namespace gz
