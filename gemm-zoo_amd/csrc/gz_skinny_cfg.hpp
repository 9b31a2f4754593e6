// Host-side geometry of the weight-streaming (skinny M) rung, shared by the
// launcher and gz_plan.
#pragma once

#include "../../include/gemm_zoo.h"

namespace gz {

constexpr int SKINNY_MAX_M = 128;      // most rows of activations the streaming kernels take
constexpr int SKINNY_REG_MAX_M = 16;   // above: activations are shared through LDS (stream_tile_kernel)
constexpr int SKINNY_COLS_PER_WAVE = 16;
constexpr int SKINNY_K_STEP = 64;      // elements of K consumed per super-step (128 bytes per weight row)
// direct-to-LDS kernel: 128-element K chunks, 32 rows x 256 bytes per stage, waves per work-group, stages per wave
constexpr int SKINNY_DTL_K_STEP = 128;
constexpr int SKINNY_DTL_STAGE_BYTES = 8192;
constexpr int SKINNY_DTL_WAVES = 4;
constexpr int SKINNY_DTL_STAGES = 2;
// producer / consumer tile kernel: 64 K elements (128-byte rows) per stage, at most 64 columns per work-group,
// four consumer and four producer waves, ring depth by number of 32-row blocks of A
constexpr int STREAM_TILE_K_STEP = 64;
constexpr int STREAM_TILE_ROW_BYTES = 128;
constexpr int STREAM_TILE_COLS = 64;
constexpr int STREAM_TILE_THREADS = 512;
constexpr int STREAM_TILE_STAGES_1 = 8, STREAM_TILE_STAGES_2 = 4, STREAM_TILE_STAGES_4 = 4;

// the same with wide column blocks and a split K (65 ... 128 rows, long K): 64 CB columns per work-group, CB = 2 ... 4,
// ring depth by CB; a work-group's partial sums are 4 waves x 2 row blocks x CB column blocks x 4 KiB
constexpr int STREAM_WIDE_MIN_K = 8192;
constexpr int STREAM_WIDE_MAX_CB = 4;
constexpr int STREAM_WIDE_STAGES_2 = 4, STREAM_WIDE_STAGES_3 = 3, STREAM_WIDE_STAGES_4 = 3;
inline int stream_wide_stages(int cb) { return cb == 2 ? STREAM_WIDE_STAGES_2 : cb == 3 ? STREAM_WIDE_STAGES_3 : STREAM_WIDE_STAGES_4; }
inline long long stream_wide_slot_bytes(int cb) { return 4LL * 2 * cb * 4 * 1024; }

enum { SKINNY_KIND_REG = 0, SKINNY_KIND_DTL = 1, SKINNY_KIND_TILE = 2, SKINNY_KIND_TILE_WIDE = 3 };

struct SkinnyCfg {
  int mb;             // rows of A the kernel instance covers: 16, 32, 64 or 128
  int cols_per_wave;  // 16
  int waves;          // wavefronts per work-group
  int cols_per_wg;
  int threads;
  int grid_n;         // work-groups along N
  int split_k;        // K slices (partial sums reduced by a second kernel when > 1)
  int k_per_split;
  int kind;           // SKINNY_KIND_*
  int lds_bytes;
  int cb;             // SKINNY_KIND_TILE_WIDE: 64-column blocks per work-group
  long long workspace_bytes;   // partial sums of a split K (0: none)
};

// Decode-shaped problems only: 16-bit float inputs, activations row-major (K
// contiguous), weights column-major (K contiguous), whole K super-steps.
inline bool skinny_supported(int types, int M, int N, int K, int layoutA, int layoutB) {
  if (types != GZ_BF16BF16F32 && types != GZ_BF16BF16BF16 && types != GZ_F16F16F16) return false;
  if (layoutA != GZ_ROW_MAJOR || layoutB != GZ_COL_MAJOR) return false;
  if (M < 1 || M > SKINNY_MAX_M || N < 1 || K < SKINNY_K_STEP) return false;
  if ((long long)K * 2 * SKINNY_MAX_M >= (1LL << 32)) return false;  // rows are addressed with 32-bit byte offsets
  return K % SKINNY_K_STEP == 0;
}

// The streaming kernels copy 16-byte pieces of the rows of A and the columns of B and address them with 32-bit byte
// offsets from the first row (column of the work-group): leading dimensions of whole pieces, below 2^32 / (2 * 128).
inline bool skinny_lines_ok(long long lda, long long ldb) {
  return lda % 8 == 0 && ldb % 8 == 0 && lda * 2 * SKINNY_MAX_M < (1LL << 32) && ldb * 2 * SKINNY_MAX_M < (1LL << 32);
}

// What the launcher's own choice sends here: always the register-resident cases; the LDS-shared tile kernel only
// while the tiled MFMA rung could not give every compute unit a 128 x 128 tile of its own.
inline bool skinny_preferred(int types, int M, int N, int K, int layoutA, int layoutB, int num_cus) {
  if (!skinny_supported(types, M, N, K, layoutA, layoutB)) return false;
  if (num_cus <= 0) num_cus = 256;
  return M <= 32 || (long long)((N + 127) / 128) <= num_cus;
}

// equal column groups, one or more per compute unit, at most max_cols columns and a multiple of 4 each
inline int skinny_balanced_cols(int N, int num_cus, int max_cols) {
  if (num_cus <= 0) num_cus = 256;
  for (int w = 1; w <= 1024; w++) {
    const long long slots = (long long)num_cus * w;
    int per = (int)((N + slots - 1) / slots);
    per = (per + 3) / 4 * 4;
    if (per <= max_cols) return per;
  }
  return max_cols;
}

// Wide column blocks with a split K.  With 64 columns per work-group every compute unit pulls ALL of A from its L2
// beside its share of B, and at 65 ... 128 rows that, not HBM, sets the time (M = 128, N = 14336, K = 8192: 2 MiB of A
// and 0.9 MiB of B per compute unit, 60 us where the B stream alone is 42 at the 5.6 TB/s this part streams).  What a work-group takes in of A is
// rows x its K range, whatever its columns: splitting K in KS parts AND widening the column blocks KS-fold keeps one
// work-group per compute unit and divides the A traffic by KS.  The partial sums go to a workspace in the order the
// waves hold them (whole 1 KiB stores) and a second launch adds them in the order of the K parts - a fixed order, no
// waiting - and applies alpha, beta and the rounding.  Taken for 64 < M <= 128 from K = 8192 on where the column
// blocks come out at 65 ... 256 columns and the workspace fits.  The first launch then runs at the rate of the B
// stream (M = 128, N = 14336: 43 us at K = 8192, 75 at 14336); the second costs 8 us: 60.1 -> 53.9 us and
// 108.5 -> 83.1.
inline bool skinny_resolve_wide(int M, int N, int K, int num_cus, unsigned long long ws_limit, int* split, int* cols) {
  if (num_cus <= 0) num_cus = 256;
  if (M <= 64 || M > SKINNY_MAX_M || K < STREAM_WIDE_MIN_K) return false;
  // four parts where the column blocks allow it, else two (M = 128, N = 14336, us, two / four parts: K = 8192
  // 56.0 / 56.3, K = 14336 93.9 / 84.5, before the second launch wrote whole rows; at K = 4096 the split loses to the one-launch kernel, 34.2 against 31.6)
  for (int ks = 4; ks >= 2; ks >>= 1) {
    if (num_cus % ks || (K / STREAM_TILE_K_STEP) < 8 * ks) continue;
    const int groups = num_cus / ks;
    int per = (N + groups - 1) / groups;
    per = (per + 3) / 4 * 4;
    if (per <= STREAM_TILE_COLS || per > STREAM_TILE_COLS * STREAM_WIDE_MAX_CB) continue;
    const int cb = (per + STREAM_TILE_COLS - 1) / STREAM_TILE_COLS;
    const long long grid_n = (N + per - 1) / per;
    if ((unsigned long long)(grid_n * ks * stream_wide_slot_bytes(cb)) > ws_limit) continue;
    *split = ks;
    *cols = per;
    return true;
  }
  return false;
}

inline SkinnyCfg skinny_resolve(int M, int N, int K, int num_cus, unsigned long long ws_limit = ~0ULL) {
  SkinnyCfg c;
  c.split_k = 1;
  c.k_per_split = K;
  c.cb = 1;
  c.workspace_bytes = 0;
  int wide_split = 1, wide_cols = 0;
  if (skinny_resolve_wide(M, N, K, num_cus, ws_limit, &wide_split, &wide_cols)) {
    c.kind = SKINNY_KIND_TILE_WIDE;
    c.mb = 128;
    c.cols_per_wg = wide_cols;
    c.cb = (wide_cols + STREAM_TILE_COLS - 1) / STREAM_TILE_COLS;
    c.cols_per_wave = 32 * c.cb;
    c.waves = STREAM_TILE_THREADS / 64;
    c.split_k = wide_split;
    c.k_per_split = K / wide_split;   // (whole 64-element stages are dealt as evenly as they divide)
    c.lds_bytes = stream_wide_stages(c.cb) * (128 + STREAM_TILE_COLS * c.cb) * STREAM_TILE_ROW_BYTES;
    c.threads = c.waves * 64;
    c.grid_n = (N + c.cols_per_wg - 1) / c.cols_per_wg;
    c.workspace_bytes = (long long)c.grid_n * c.split_k * stream_wide_slot_bytes(c.cb);
    return c;
  }
  if (M > SKINNY_REG_MAX_M) {
    c.kind = SKINNY_KIND_TILE;
    c.mb = M <= 32 ? 32 : M <= 64 ? 64 : 128;
    const int stages = c.mb == 32 ? STREAM_TILE_STAGES_1 : c.mb == 64 ? STREAM_TILE_STAGES_2 : STREAM_TILE_STAGES_4;
    c.cols_per_wg = skinny_balanced_cols(N, num_cus, STREAM_TILE_COLS);
    c.cols_per_wave = 32;
    c.waves = STREAM_TILE_THREADS / 64;
    c.lds_bytes = stages * (c.mb + STREAM_TILE_COLS) * STREAM_TILE_ROW_BYTES;
  } else if (K % SKINNY_DTL_K_STEP == 0) {
    c.kind = SKINNY_KIND_DTL;
    c.mb = 16;
    c.cols_per_wg = skinny_balanced_cols(N, num_cus, 32);
    c.cols_per_wave = c.cols_per_wg;  // every wave of the work-group works on all of its columns (K is split)
    c.waves = SKINNY_DTL_WAVES;
    c.lds_bytes = SKINNY_DTL_WAVES * SKINNY_DTL_STAGES * SKINNY_DTL_STAGE_BYTES;
  } else {
    c.kind = SKINNY_KIND_REG;
    c.mb = 16;
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
