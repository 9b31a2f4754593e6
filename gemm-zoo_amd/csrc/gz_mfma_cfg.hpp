// Host-side tile-config table of the MFMA rung (shared by the launcher and gz_plan).
#pragma once

#include <stddef.h>
#include <stdint.h>

#include "../../include/gemm_zoo.h"

namespace gz {

struct MfmaCfg {
  int id;       // variant id (1-based; 0 means "let the launcher choose")
  int bm, bn;   // work-group tile
  int waves_m, waves_n;
  int hand_scheduled;  // fast path: 0 compiler-scheduled, 1 fixed sequence / two 128-byte buffers,
                       // 2 fixed sequence / four 64-byte buffers
};

// K slab per tile row is 128 bytes whatever the element type.
constexpr int MFMA_SLAB_BYTES = 128;
constexpr int MFMA_LDS_PITCH = 144;

static const MfmaCfg kMfmaCfgs[] = {
    {1, 256, 256, 2, 2, 0},  // 4 waves of 128x128: fewest LDS bytes per MFMA
    {2, 256, 256, 2, 4, 0},  // 8 waves of 128x64: two waves per SIMD hide each other's waits
    {3, 128, 128, 2, 2, 0},  // small tile for small problems / ragged tails
    {4, 256, 128, 2, 2, 0},  // 4 waves of 128x64
    {5, 256, 256, 2, 2, 1},  // tile of variant 1 with the hand-scheduled main loop
    {6, 256, 256, 2, 2, 2},  // tile of variant 1, hand-scheduled, four-buffer pipeline
    {7, 256, 256, 2, 4, 2},  // tile of variant 2 (8 waves), hand-scheduled, four-buffer pipeline
};
constexpr int kNumMfmaCfgs = (int)(sizeof(kMfmaCfgs) / sizeof(kMfmaCfgs[0]));

inline int mfma_lds_bytes(const MfmaCfg& c) { return 2 * (c.bm + c.bn) * MFMA_LDS_PITCH; }

// How a problem sits on a tile configuration (16-byte alignment of the pointers is the caller's to check):
//   WHOLE      whole tiles and whole K slabs
//   RAGGED_MN  whole K slabs, row-major A, rows of A and B a whole number of 16-byte pieces, but M or N not a
//              multiple of the tile: the 256x256 direct-to-LDS kernels handle it by clamping rows
//   GENERAL    everything else: the predicated kernel
enum { MFMA_SHAPE_WHOLE = 0, MFMA_SHAPE_RAGGED_MN = 1, MFMA_SHAPE_GENERAL = 2 };
inline int mfma_shape_class(const MfmaCfg& c, int in_size, int M, int N, int K, int layoutA, int layoutB) {
  const int bk = MFMA_SLAB_BYTES / in_size, epv = 16 / in_size;
  if (K <= 0 || K % bk) return MFMA_SHAPE_GENERAL;
  if (M % c.bm == 0 && N % c.bn == 0) return MFMA_SHAPE_WHOLE;
  if (layoutA != GZ_ROW_MAJOR) return MFMA_SHAPE_GENERAL;
  if (layoutB == GZ_ROW_MAJOR && N % epv) return MFMA_SHAPE_GENERAL;
  return MFMA_SHAPE_RAGGED_MN;
}
inline bool mfma_whole_tiles(const MfmaCfg& c, int in_size, int M, int N, int K) {
  return mfma_shape_class(c, in_size, M, N, K, GZ_ROW_MAJOR, GZ_COL_MAJOR) == MFMA_SHAPE_WHOLE;
}

// Picks the tile configuration by an estimate of the launch's duration:
//     rounds of tiles over the compute units  x  tile area  x  penalty of the tile shape  x  penalty of the kernel
// A 256x256 tile needs the fewest bytes per flop and runs the hand-scheduled kernels, but a grid that does not
// fill the device, or that leaves a nearly empty last round (N = 4097: 17 tile columns for one column of data),
// is better served by smaller tiles.  The penalties are measured on MI355X (fp16 4095x4097x1023: 256x256 255 us,
// 256x128 174 us, 128x128 156 us; 4096x4352x1024 row/row: 256x256 hand-scheduled 79 us, 128x128 general 103 us;
// bf16 2048^3 row/col: 128x128 30 us, 256x128 41 us, 256x256 51 us).
//   bf16 4096^3 (interleaved runs, us)  v1 117  v2 109  v5 108  v6 109  v7 106
//   bf16 8192^3                         v1 904  v2 865  v6 845  v7 885
//   int8 8192^3                         v1 543  v2 558  v5 579  v6 536  v7 582
// Direct-to-LDS kernels exist for row-major A with whole tiles: hand-scheduled for 256x256 (column-major B: both
// wave shapes; row-major B: four waves), compiler-scheduled for the smaller tiles; on any other problem the same
// tile runs the general kernel, so choosing them is always safe.
inline bool mfma_resolve(int types, int M, int N, int K, int layoutA, int layoutB, int variant, int num_cus,
                         MfmaCfg* out) {
  if (variant < 0 || variant > kNumMfmaCfgs) return false;
  if (variant > 0) {
    *out = kMfmaCfgs[variant - 1];
    return true;
  }
  if (num_cus <= 0) num_cus = 256;
  const int in_size = (types == GZ_S8S8S32 || types == GZ_E4M3E4M3F16 || types == GZ_E5M2E5M2F16) ? 1 : types == GZ_F32F32F32 ? 4 : 2;
  const bool a_rows = layoutA == GZ_ROW_MAJOR, b_cols = layoutB == GZ_COL_MAJOR;
  // candidates: 256x256 (id 6), 256x128 (id 4), 128x128 (id 3)
  const int cand[3] = {5, 3, 2};
  const double shape_pen[3] = {1.0, 1.1, 1.25};
  double best = 0;
  int pick = 5;
  for (int i = 0; i < 3; i++) {
    const MfmaCfg& c = kMfmaCfgs[cand[i]];
    const long long tiles = (long long)((M + c.bm - 1) / c.bm) * ((N + c.bn - 1) / c.bn);
    const long long rounds = (tiles + num_cus - 1) / num_cus;
    // whole tiles: every candidate has a direct-to-LDS kernel; ragged M or N: the 256x256 ones only
    const int cls = mfma_shape_class(c, in_size, M, N, K, layoutA, layoutB);
    const bool direct = a_rows && types != GZ_F32F32F32 &&
                        (cls == MFMA_SHAPE_WHOLE || (cls == MFMA_SHAPE_RAGGED_MN && i == 0));
    const double cost = (double)rounds * c.bm * c.bn * shape_pen[i] * (direct ? 1.0 : 2.2);
    if (i == 0 || cost < best) {
      best = cost;
      pick = cand[i];
    }
  }
  *out = kMfmaCfgs[pick];
  if (pick == 5 && (types == GZ_BF16BF16F32 || types == GZ_BF16BF16BF16 || types == GZ_F16F16F16) && a_rows && b_cols) {  // 16-bit, K-contiguous B: eight waves while the grid is small
    const long long tiles = (long long)((M + 255) / 256) * ((N + 255) / 256);
    if (tiles <= 2LL * num_cus) *out = kMfmaCfgs[6];
  }
  return true;
}

// Shape class of a launch: the direct-to-LDS kernels also need 16-byte aligned operands.
inline int mfma_launch_class(const MfmaCfg& c, int in_size, int M, int N, int K, int layoutA, int layoutB, const void* A,
                             const void* B, const void* C, const void* D) {
  const uintptr_t bits = (uintptr_t)A | (uintptr_t)B | (uintptr_t)C | (uintptr_t)D;
  if (bits & 15u) return MFMA_SHAPE_GENERAL;
  return mfma_shape_class(c, in_size, M, N, K, layoutA, layoutB);
}

}  // namespace gz
