// Host-side geometry of the weight-streaming (skinny M) rung, shared by the
// launcher and gz_plan.
#pragma once

#include "../../include/gemm_zoo.h"

namespace gz {

constexpr int SKINNY_MAX_M = 32;       // rows of activations the streaming kernel keeps per wave
constexpr int SKINNY_COLS_PER_WAVE = 16;
constexpr int SKINNY_K_STEP = 64;      // elements of K consumed per super-step (128 bytes per weight row)

struct SkinnyCfg {
  int mb;             // rows padded to a multiple of 16
  int cols_per_wave;  // 16
  int waves;          // wavefronts per work-group
  int cols_per_wg;
  int threads;
  int grid_n;         // work-groups along N
  int split_k;        // K slices (partial sums reduced by a second kernel when > 1)
  int k_per_split;
};

// Decode-shaped problems only: 16-bit float inputs, activations row-major (K
// contiguous), weights column-major (K contiguous), whole K super-steps.
inline bool skinny_supported(int types, int M, int N, int K, int layoutA, int layoutB) {
  if (types == GZ_S8S8S32) return false;
  if (layoutA != GZ_ROW_MAJOR || layoutB != GZ_COL_MAJOR) return false;
  if (M < 1 || M > SKINNY_MAX_M || N < 1 || K < SKINNY_K_STEP) return false;
  return K % SKINNY_K_STEP == 0;
}

inline SkinnyCfg skinny_resolve(int M, int N, int K, int /*num_cus*/) {
  SkinnyCfg c;
  c.mb = M <= 16 ? 16 : 32;
  c.cols_per_wave = SKINNY_COLS_PER_WAVE;
  c.waves = 2;
  c.cols_per_wg = c.cols_per_wave * c.waves;
  c.threads = c.waves * 64;
  c.grid_n = (N + c.cols_per_wg - 1) / c.cols_per_wg;
  c.split_k = 1;
  c.k_per_split = K;
  return c;
}

}  // namespace gz
