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

// Picks the tile configuration.  A 256x256 tile needs the fewest bytes per flop;
// it is kept as long as the grid still covers every compute unit, otherwise the
// tile shrinks so that more work-groups exist.
inline bool mfma_resolve(int types, int M, int N, int /*K*/, int layoutA, int layoutB, int variant, int num_cus,
                         MfmaCfg* out) {
  if (variant < 0 || variant > kNumMfmaCfgs) return false;
  if (variant > 0) {
    *out = kMfmaCfgs[variant - 1];
    return true;
  }
  auto tiles = [&](const MfmaCfg& c) {
    return (long long)((M + c.bm - 1) / c.bm) * ((N + c.bn - 1) / c.bn);
  };
  // Measured on MI355X (interleaved runs, us): bf16 4096^3  v1 117  v2 109  v5 108  v6 109  v7 106
  //                                           bf16 8192^3  v1 904  v2 865  v6 845  v7 885
  //                                           int8 8192^3  v1 543  v2 558  v5 579  v6 536  v7 582
  // The hand-scheduled kernels only exist for K-contiguous operands and whole tiles; on any other problem
  // the same tile runs the general kernel, so choosing them here is always safe.
  // Row-major B (with row-major A) has its hand-scheduled kernel in the four-wave form only: each B fragment
  // takes two transposing LDS reads, which fit the instruction slots of 16 MFMAs per step but not of 8.
  const bool b_rows = layoutA == GZ_ROW_MAJOR && layoutB == GZ_ROW_MAJOR;
  if (tiles(kMfmaCfgs[0]) >= num_cus) {
    if (types == 0 || b_rows) *out = kMfmaCfgs[5];                        // 4 waves, four-buffer pipeline
    else *out = tiles(kMfmaCfgs[0]) <= 2 * num_cus ? kMfmaCfgs[6] : kMfmaCfgs[5];
  }
  else if (tiles(kMfmaCfgs[3]) >= num_cus) *out = kMfmaCfgs[3];
  else *out = kMfmaCfgs[2];
  return true;
}

// The unpredicated kernel needs whole tiles, whole K slabs and 16-byte aligned
// operands; everything else runs the predicated (edge) instantiation.
inline bool mfma_needs_edge(const MfmaCfg& c, int in_size, int /*out_size*/, int M, int N, int K, const void* A,
                            const void* B, const void* C, const void* D) {
  const int bk = MFMA_SLAB_BYTES / in_size;
  if (K == 0 || M % c.bm || N % c.bn || K % bk) return true;
  const uintptr_t bits = (uintptr_t)A | (uintptr_t)B | (uintptr_t)C | (uintptr_t)D;
  return (bits & 15u) != 0;
}

}  // namespace gz
