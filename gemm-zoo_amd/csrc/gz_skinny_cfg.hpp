// Host-side geometry of the weight-streaming (skinny M) rung, shared by the
// launcher and gz_plan.
#pragma once

#include "../../include/gemm_zoo.h"

namespace gz {

constexpr int SKINNY_MAX_M = 32;       // rows of activations the streaming kernel keeps per wave
constexpr int SKINNY_COLS_PER_WAVE = 16;
constexpr int SKINNY_K_STEP = 64;      // elements of K consumed per super-step (128 bytes per weight row)
// direct-to-LDS kernel: 128-element K chunks, 32 rows x 256 bytes per stage, waves per work-group, stages per wave
constexpr int SKINNY_DTL_K_STEP = 128;
constexpr int SKINNY_DTL_STAGE_BYTES = 8192;
constexpr int SKINNY_DTL_WAVES = 4;
constexpr int SKINNY_DTL_STAGES = 2;

struct SkinnyCfg {
  int mb;             // rows padded to a multiple of 16
  int cols_per_wave;  // 16
  int waves;          // wavefronts per work-group
  int cols_per_wg;
  int threads;
  int grid_n;         // work-groups along N
  int split_k;        // K slices (partial sums reduced by a second kernel when > 1)
  int k_per_split;
  int dtl;            // 1: direct-to-LDS kernel (K % 128 == 0), 0: register-streaming kernel
  int lds_bytes;
};

// Decode-shaped problems only: 16-bit float inputs, activations row-major (K
// contiguous), weights column-major (K contiguous), whole K super-steps.
inline bool skinny_supported(int types, int M, int N, int K, int layoutA, int layoutB) {
  if (types == GZ_S8S8S32) return false;
  if (layoutA != GZ_ROW_MAJOR || layoutB != GZ_COL_MAJOR) return false;
  if (M < 1 || M > SKINNY_MAX_M || N < 1 || K < SKINNY_K_STEP) return false;
  return K % SKINNY_K_STEP == 0;
}

inline SkinnyCfg skinny_resolve(int M, int N, int K, int num_cus) {
  SkinnyCfg c;
  c.mb = M <= 16 ? 16 : 32;
  c.split_k = 1;
  c.k_per_split = K;
  c.dtl = K % SKINNY_DTL_K_STEP == 0;
  if (c.dtl) {
    // equal column groups, one or more per compute unit, at most 32 columns and a multiple of 4 each
    if (num_cus <= 0) num_cus = 256;
    int cols = 32;
    for (int w = 1; w <= 64; w++) {
      const long long slots = (long long)num_cus * w;
      int per = (int)((N + slots - 1) / slots);
      per = (per + 3) / 4 * 4;
      if (per <= 32) {
        cols = per;
        break;
      }
    }
    c.cols_per_wave = cols;          // every wave of the work-group works on all of its columns (K is split)
    c.waves = SKINNY_DTL_WAVES;
    c.cols_per_wg = cols;
    c.lds_bytes = SKINNY_DTL_WAVES * SKINNY_DTL_STAGES * SKINNY_DTL_STAGE_BYTES;
  } else {
    c.cols_per_wave = SKINNY_COLS_PER_WAVE;
    c.waves = 2;
    c.cols_per_wg = c.cols_per_wave * c.waves;
    c.lds_bytes = 0;
  }
  c.threads = c.waves * 64;
  c.grid_n = (N + c.cols_per_wg - 1) / c.cols_per_wg;
  return c;
}

}  // namespace gz
