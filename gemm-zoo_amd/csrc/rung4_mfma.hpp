// Rung 4: wavefront-level MFMA GEMM for gfx950.
//
// One work-group owns a BM x BN tile of D and walks K in slabs of 128 bytes per
// row (64 16-bit elements or 128 int8).  Both operand slabs live in LDS as
// [row][k] with a 16-byte pad per row (pitch 144 B), which makes the 128-bit
// fragment reads of 16 consecutive rows hit 16 distinct 4-bank groups.
// Each lane's MFMA operand is 16 contiguous K-bytes of one row, so a fragment
// is a single ds_read_b128 whatever the element type:
//     v_mfma_f32_32x32x16_{bf16,f16}  (8 elements / lane)
//     v_mfma_i32_32x32x32_i8          (16 elements / lane)
// Operands whose contiguous dimension is not K (row-major B, column-major A)
// are transposed in registers on their way into LDS.
// The B fragment is passed as the instruction's first operand, so every lane
// ends up with 4 consecutive columns of one output row and the epilogue stores
// are 128-bit (fp32 / int32) or 64-bit (16-bit outputs).
//
// Stands in for nvidia/kernels/sm_80/{bf16,fp16}_mma_gemm.cuh and
// intel/kernels/xe_gemm_*_m8k16.hpp (same operation, new design).
#pragma once
#include "gz_common.hpp"
#include "gz_mfma_cfg.hpp"

namespace gz {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));
typedef int i32x16_t __attribute__((ext_vector_type(16)));
typedef int i32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));

template <int TYPES> struct AccVec { using type = f32x16_t; };
template <> struct AccVec<GZ_S8S8S32> { using type = i32x16_t; };

template <int TYPES>
__device__ inline typename AccVec<TYPES>::type mfma32(u32x4_t first, u32x4_t second,
                                                      typename AccVec<TYPES>::type acc) {
  if constexpr (TYPES == GZ_S8S8S32) {
    return __builtin_amdgcn_mfma_i32_32x32x32_i8(__builtin_bit_cast(i32x4_t, first),
                                                 __builtin_bit_cast(i32x4_t, second), acc, 0, 0, 0);
  } else if constexpr (TYPES == GZ_F16F16F16) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8_t, first),
                                                  __builtin_bit_cast(f16x8_t, second), acc, 0, 0, 0);
  } else {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, first),
                                                   __builtin_bit_cast(bf16x8_t, second), acc, 0, 0, 0);
  }
}

constexpr int SLAB_BYTES = 128;           // K bytes per tile row per slab
constexpr int PITCH = SLAB_BYTES + 16;    // LDS row pitch
constexpr int KSTEPS = SLAB_BYTES / 32;   // MFMA steps per slab

// 16-byte global load of `EPV` elements starting at element (line, pos) of a
// matrix whose lines are `extent` long.  With EDGE the access is predicated and
// zero-filled, and may be unaligned (gfx950 global loads tolerate that).
template <typename in_t, bool EDGE>
__device__ inline u32x4_t load16(const in_t* __restrict__ base, int line, int lines, int pos, int extent) {
  constexpr int EPV = 16 / (int)sizeof(in_t);
  if constexpr (!EDGE) {
    return *reinterpret_cast<const u32x4_t*>(base + (size_t)line * extent + pos);
  } else {
    u32x4_t v = {0u, 0u, 0u, 0u};
    if (line < lines) {
      const in_t* p = base + (size_t)line * extent + pos;
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

  // rows_total: M or N ; row0: first tile row ; k0: first k of the slab
  __device__ inline void load(const in_t* __restrict__ base, int rows_total, int K, int row0, int k0, int tid) {
    if constexpr (KC) {
#pragma unroll
      for (int it = 0; it < VECS; it++) {
        const int id = it * NT + tid;
        const int row = id >> 3, c = id & 7;
        r[it] = load16<in_t, EDGE>(base, row0 + row, rows_total, k0 + c * EPV, K);
      }
    } else {
      constexpr int MC = ROWS / EPV;  // 16-byte columns across the tile
#pragma unroll
      for (int u = 0; u < UNITS; u++) {
        const int id = u * NT + tid;
        const int mc = id % MC, ku = id / MC;
#pragma unroll
        for (int t = 0; t < TR; t++)
          r[u * TR + t] = load16<in_t, EDGE>(base, k0 + ku * TR + t, K, row0 + mc * EPV, rows_total);
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
      constexpr int MC = ROWS / EPV;
#pragma unroll
      for (int u = 0; u < UNITS; u++) {
        const int id = u * NT + tid;
        const int mc = id % MC, ku = id / MC;
        char* dst = lds + (mc * EPV) * PITCH + ku * 4;
        if constexpr (ES == 2) {
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
__device__ inline void tile_of_block(int bid, int tiles_m, int tiles_n, int& tm, int& tn) {
  constexpr int XCDS = 8, GROUP_M = 4;
  const int total = tiles_m * tiles_n;
  const int per = total / XCDS, rem = total % XCDS;
  const int xcd = bid % XCDS, idx = bid / XCDS;
  int lid = xcd * per + (xcd < rem ? xcd : rem) + idx;
  const int band = GROUP_M * tiles_n;
  const int b = lid / band;
  const int first_m = b * GROUP_M;
  const int rows = (tiles_m - first_m) < GROUP_M ? (tiles_m - first_m) : GROUP_M;
  const int in_band = lid - b * band;
  tm = first_m + in_band % rows;
  tn = in_band / rows;
}

template <int TYPES, int BM, int BN, int WAVES_M, int WAVES_N, bool A_KC, bool B_KC, bool EDGE>
__global__ void __launch_bounds__(WAVES_M* WAVES_N * 64)
    mfma_gemm_kernel(GemmArgs<TYPES> g, int tiles_m, int tiles_n) {
  using T = Traits<TYPES>;
  using in_t = typename T::in_t;
  using out_t = typename T::out_t;
  using acc_v = typename AccVec<TYPES>::type;
  constexpr int NT = WAVES_M * WAVES_N * 64;
  constexpr int ES = (int)sizeof(in_t);
  constexpr int BK = SLAB_BYTES / ES;
  constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;
  constexpr int FM = WM / 32, FN = WN / 32;
  static_assert(WM % 32 == 0 && WN % 32 == 0, "wave tile must be a multiple of the 32x32 MFMA block");
  constexpr int A_BYTES = BM * PITCH, B_BYTES = BN * PITCH;
  constexpr int STAGE_BYTES = A_BYTES + B_BYTES;

  extern __shared__ __attribute__((aligned(16))) char lds[];

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int wm = wave % WAVES_M, wn = wave / WAVES_M;
  int tm, tn;
  tile_of_block(blockIdx.x, tiles_m, tiles_n, tm, tn);
  const int m0 = tm * BM, n0 = tn * BN;

  Stager<in_t, BM, NT, A_KC, EDGE> sa;
  Stager<in_t, BN, NT, B_KC, EDGE> sb;

  acc_v acc[FM][FN];
#pragma unroll
  for (int i = 0; i < FM; i++)
#pragma unroll
    for (int j = 0; j < FN; j++)
#pragma unroll
      for (int v = 0; v < 16; v++) acc[i][j][v] = 0;

  const int ktiles = (g.K + BK - 1) / BK;

  sa.load(g.A, g.M, g.K, m0, 0, tid);
  sb.load(g.B, g.N, g.K, n0, 0, tid);
  sa.store(lds, tid);
  sb.store(lds + A_BYTES, tid);
  __syncthreads();

  // fragment base offsets of this lane inside a stage
  const int frag_row = lane & 31, frag_k = (lane >> 5) * 16;
  const int a_off = (wm * WM + frag_row) * PITCH + frag_k;
  const int b_off = A_BYTES + (wn * WN + frag_row) * PITCH + frag_k;

  for (int kt = 0; kt < ktiles; kt++) {
    const char* cur = lds + (kt & 1) * STAGE_BYTES;
    char* nxt = lds + ((kt + 1) & 1) * STAGE_BYTES;
    const bool more = kt + 1 < ktiles;
    if (more) {
      sa.load(g.A, g.M, g.K, m0, (kt + 1) * BK, tid);
      sb.load(g.B, g.N, g.K, n0, (kt + 1) * BK, tid);
    }
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ks++) {
      u32x4_t af[FM], bf[FN];
#pragma unroll
      for (int i = 0; i < FM; i++)
        af[i] = *reinterpret_cast<const u32x4_t*>(cur + a_off + i * 32 * PITCH + ks * 32);
#pragma unroll
      for (int j = 0; j < FN; j++)
        bf[j] = *reinterpret_cast<const u32x4_t*>(cur + b_off + j * 32 * PITCH + ks * 32);
#pragma unroll
      for (int i = 0; i < FM; i++)
#pragma unroll
        for (int j = 0; j < FN; j++) acc[i][j] = mfma32<TYPES>(bf[j], af[i], acc[i][j]);
    }
    if (more) {
      sa.store(nxt, tid);
      sb.store(nxt + A_BYTES, tid);
    }
    __syncthreads();
  }

  // Epilogue.  acc[i][j][4*q + e] is D(m, n + e) with
  //   m = m0 + wm*WM + 32 i + lane%32,  n = n0 + wn*WN + 32 j + 8 q + 4 (lane/32).
  const int N = g.N;
  const bool use_c = g.beta != 0;
#pragma unroll
  for (int i = 0; i < FM; i++) {
    const int m = m0 + wm * WM + 32 * i + (lane & 31);
#pragma unroll
    for (int j = 0; j < FN; j++) {
#pragma unroll
      for (int q = 0; q < 4; q++) {
        const int n = n0 + wn * WN + 32 * j + 8 * q + 4 * (lane >> 5);
        const size_t o = (size_t)m * N + n;
        if constexpr (!EDGE) {
          out_t cv[4] = {0, 0, 0, 0}, dv[4];
          if (use_c) __builtin_memcpy(cv, g.C + o, sizeof(cv));
#pragma unroll
          for (int e = 0; e < 4; e++) dv[e] = epilogue<TYPES>(acc[i][j][4 * q + e], g.alpha, g.beta, &cv[e]);
          if constexpr (sizeof(out_t) == 4) *reinterpret_cast<u32x4_t*>(g.D + o) = __builtin_bit_cast(u32x4_t, dv);
          else *reinterpret_cast<u32x2_t*>(g.D + o) = __builtin_bit_cast(u32x2_t, dv);
        } else {
          if (m < g.M) {
#pragma unroll
            for (int e = 0; e < 4; e++)
              if (n + e < N) g.D[o + e] = epilogue<TYPES>(acc[i][j][4 * q + e], g.alpha, g.beta, g.C + o + e);
          }
        }
      }
    }
  }
}

// ---------------------------------------------------------------------------
// Launcher
// ---------------------------------------------------------------------------
template <int TYPES, int BM, int BN, int WAVES_M, int WAVES_N>
static int launch_cfg(const GemmArgs<TYPES>& g, bool edge, hipStream_t s) {
  const int tiles_m = ceil_div(g.M, BM), tiles_n = ceil_div(g.N, BN);
  const dim3 grid((unsigned)(tiles_m * tiles_n)), block(WAVES_M * WAVES_N * 64);
  const size_t lds = 2u * (size_t)(BM + BN) * PITCH;
  const bool akc = g.layoutA == GZ_ROW_MAJOR, bkc = g.layoutB == GZ_COL_MAJOR;

#define GZ_LAUNCH(AKC, BKC, EDGE)                                                                   \
  do {                                                                                              \
    auto kern = mfma_gemm_kernel<TYPES, BM, BN, WAVES_M, WAVES_N, AKC, BKC, EDGE>;                   \
    GZ_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(kern),                             \
                                   hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));          \
    hipLaunchKernelGGL(kern, grid, block, lds, s, g, tiles_m, tiles_n);                             \
  } while (0)

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

template <int TYPES> int launch_mfma(const GemmArgs<TYPES>& g, int variant, hipStream_t s) {
  using in_t = typename Traits<TYPES>::in_t;
  MfmaCfg cfg;
  if (!mfma_resolve(TYPES, g.M, g.N, g.K, variant, 256, &cfg)) {
    set_error("mfma rung: unknown variant %d", variant);
    return GZ_ERR_UNSUPPORTED;
  }
  const bool edge = mfma_needs_edge(cfg, (int)sizeof(in_t), (int)sizeof(typename Traits<TYPES>::out_t), g.M, g.N,
                                    g.K, g.A, g.B, g.C, g.D);
  switch (cfg.id) {
    case 1: return launch_cfg<TYPES, 256, 256, 2, 2>(g, edge, s);
    case 2: return launch_cfg<TYPES, 256, 256, 2, 4>(g, edge, s);
    case 3: return launch_cfg<TYPES, 128, 128, 2, 2>(g, edge, s);
    case 4: return launch_cfg<TYPES, 256, 128, 2, 2>(g, edge, s);
    default: break;
  }
  set_error("mfma rung: variant %d not built", cfg.id);
  return GZ_ERR_UNSUPPORTED;
}

}  // namespace gz
