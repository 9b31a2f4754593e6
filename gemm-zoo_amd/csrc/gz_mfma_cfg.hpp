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
  int ring;     // 0: the compiler-scheduled kernels (register-staged, or direct-to-LDS where one exists for the tile);
                // 1: the hand-scheduled ring kernel wherever the problem allows it, persistent past one round of
                //    the compute units; 2: the same kernel with one work-group per tile
  bool stream_k;  // the tiles past the last whole round of the compute units are cut along K (see mfma_plan_streamk)
};

// K slab per tile row is 128 bytes whatever the element type.
constexpr int MFMA_SLAB_BYTES = 128;
constexpr int MFMA_LDS_PITCH = 144;

static const MfmaCfg kMfmaCfgs[] = {
    {1, 256, 256, 2, 2, 0, false},   // 4 waves of 128x128: fewest LDS bytes per MFMA
    {2, 256, 256, 2, 4, 0, false},   // 8 waves of 128x64: two waves per SIMD hide each other's waits
    {3, 128, 128, 2, 2, 0, false},   // small tile for small problems / ragged tails
    {4, 256, 128, 2, 2, 0, false},   // 4 waves of 128x64
    {5, 256, 256, 2, 2, 1, false},   // tile of variant 1, hand-scheduled: ring of five buffers, 16x16 matrix instructions
    {6, 256, 256, 2, 4, 1, false},   // tile of variant 2 (8 waves), the same
    {7, 256, 256, 2, 2, 1, true},    // variant 5 with the stream-K decomposition wherever it applies
    {8, 256, 256, 2, 4, 1, true},    // variant 6, the same
    {9, 256, 256, 2, 2, 2, false},   // variant 5 with one work-group per tile (for comparisons with the persistent launch)
    {10, 256, 256, 2, 4, 2, false},  // variant 6, the same
    {11, 128, 128, 2, 2, 2, false},  // tile of variant 3 on the ring kernel, two work-groups per compute unit
    {12, 64, 64, 2, 2, 0, false},    // four waves of 32x32: grids that 128x128 tiles leave mostly empty
};
constexpr int kNumMfmaCfgs = (int)(sizeof(kMfmaCfgs) / sizeof(kMfmaCfgs[0]));
// variant 12 for 8-bit elements: the same tile on two waves of 64x32 (the transposing stores of 8-bit elements need four 16-byte
// pieces per lane and operand, which 128 lanes have on this tile and 256 do not)
static const MfmaCfg kMfmaCfg64Int8 = {12, 64, 64, 1, 2, 0, false};
// positions in the table
enum { MFMA_CFG_256_W4 = 0, MFMA_CFG_256_W8 = 1, MFMA_CFG_128 = 2, MFMA_CFG_256x128 = 3, MFMA_CFG_RING_W4 = 4,
       MFMA_CFG_RING_W8 = 5, MFMA_CFG_RING_128 = 10, MFMA_CFG_64 = 11 };
enum { MFMA_VARIANT_RING_W4 = 5, MFMA_VARIANT_RING_W8 = 6, MFMA_VARIANT_STREAMK_W4 = 7, MFMA_VARIANT_STREAMK_W8 = 8 };

// the most any kernel of the configuration asks for: the ring kernel keeps five buffers of half a slab each
inline int mfma_lds_bytes(const MfmaCfg& c) {
  return c.ring ? 5 * (c.bm + c.bn) * 64 : 2 * (c.bm + c.bn) * MFMA_LDS_PITCH;
}

// How a problem sits on a tile configuration (16-byte alignment of the pointers is the caller's to check):
//   WHOLE      whole tiles and whole K slabs
//   RAGGED_MN  whole K slabs, row-major A, rows of A and B a whole number of 16-byte pieces, but M or N not a
//              multiple of the tile: the 256x256 direct-to-LDS kernels handle it by clamping rows
//   GENERAL    everything else: the predicated kernel
enum { MFMA_SHAPE_WHOLE = 0, MFMA_SHAPE_RAGGED_MN = 1, MFMA_SHAPE_GENERAL = 2 };
inline int mfma_shape_class(const MfmaCfg& c, int in_size, int M, int N, int K, int layoutA, int layoutB) {
  const int bk = MFMA_SLAB_BYTES / in_size, epv = 16 / in_size;
  if (K <= 0 || K % bk) return MFMA_SHAPE_GENERAL;
  // the direct-to-LDS kernels address a tile's rows with 32-bit byte offsets from the tile's first row
  if ((long long)K * in_size * 256 >= (1LL << 32) || (long long)N * in_size * 256 >= (1LL << 32)) return MFMA_SHAPE_GENERAL;
  if (M % c.bm == 0 && N % c.bn == 0) return MFMA_SHAPE_WHOLE;
  // ragged M / N: lines that are not K-contiguous are clamped by whole 16-byte pieces
  if (layoutA != GZ_ROW_MAJOR && (layoutB != GZ_ROW_MAJOR || M % epv)) return MFMA_SHAPE_GENERAL;
  if (layoutB == GZ_ROW_MAJOR && N % epv) return MFMA_SHAPE_GENERAL;
  return MFMA_SHAPE_RAGGED_MN;
}
inline bool mfma_whole_tiles(const MfmaCfg& c, int in_size, int M, int N, int K) {
  return mfma_shape_class(c, in_size, M, N, K, GZ_ROW_MAJOR, GZ_COL_MAJOR) == MFMA_SHAPE_WHOLE;
}

// Picks the tile configuration by an estimate of the launch's duration, in units of one round of 256x256 tiles over
// the compute units (about 105 us at K = 4096 for bf16 on MI355X):
//     256x256   rounds                      one work-group per compute unit
//     256x128   0.75 rounds                 one work-group per compute unit, more operand bytes per flop
//     128x128   0.40 + 0.27 rounds          two work-groups share a compute unit; a lone one cannot fill it
// (rounds = tiles of that size / compute units, rounded up), times the register-staged kernel's factor (see `staged` below) where the
// problem cannot use a direct-to-LDS kernel, times 1.12 / 1.15 for the two smaller tiles on a row-major B (4096^3 row/row: 152 / 150 / 119).  A 256x256 tile needs the fewest bytes per flop and runs the hand-scheduled kernels, but a grid that does
// not fill the device, or that leaves a nearly empty last round (N = 4097: 17 tile columns for one column of data),
// is better served by smaller tiles.  Fitted to bf16 row/col squares, K = M = N (us, variants 3 / 4 / 6 =
// 128x128 / 256x128 / 256x256):
//     2048: 32 / 41 / 54     2560: 49 / 49 / 65     2816: 57 / 54 / 69     3072: 85 / 106 / 75
//     3328: 92 / 112 / 82    3584: 117 / 119 / 96   3840: 131 / 130 / 110  6144 (K 4096): 312 / 332 / 318
// and fp16 4095 x 4097 x 1023 on the predicated kernel: 112 / 143 / 153.
//   bf16 4096^3 (interleaved runs, us)  v1 117  v2 109  v5 108  v6 109  v7 106
//   bf16 8192^3                         v1 904  v2 865  v6 845  v7 885
//   int8 8192^3                         v1 543  v2 558  v5 579  v6 536  v7 582
// "Direct" here means: row-major A and whole tiles (or ragged M / N on 256x256), i.e. no predicated loads and no
// transposing stores.  256x256 then runs the hand-scheduled direct-to-LDS kernels (column-major B: both wave shapes;
// row-major B: four waves), the smaller tiles the register-staged kernel without predication (128x128 with a
// row-major B: a compiler-scheduled direct-to-LDS kernel with transposing LDS reads); on any other problem the same
// tile runs the predicated kernel, so choosing them is always safe.
inline int mfma_in_size(int types) {
  return (types == GZ_S8S8S32 || types == GZ_E4M3E4M3F16 || types == GZ_E5M2E5M2F16) ? 1 : types == GZ_F32F32F32 ? 4 : 2;
}

// Whether the stores of D carry the non-temporal hint.  Measured in interleaved runs, plain / non-temporal (us):
// outputs of 64 MiB: bf16 4096 x 4096 x {64, 1024, 4096} 17.9 / 17.5, 43.5 / 42.0, 120.2 / 119.1; several rounds of
// tiles with a long K, where the writes of one round overlap the next round's loads and no longer push operands out
// of the caches: bf16 8192^3 867 / 838, int8 8192^3 493.5 / 486.4, fp8 8192^3 415.5 / 413.7.  A launch that is
// mostly the writing of an output larger than that loses with the hint (int8 8192 x 8192 x {128, 512, 1024, 2048}
// 65 / 77, 86 / 96, 106 / 115, 158 / 163; bf16 8192 x 8192 x 256 80 / 88): the last-level cache no longer takes the
// burst in.  In between (6144^2 x 4096, int8 8192^2 x 4096) it makes no difference.
// Bit 1: the loads of C (beta != 0) carry the hint as well.  That helps only in the many-rounds case (bf16 8192^3 with
// alpha = beta = 1: 940 / 927 us, int8 561 / 548) and costs on a 64 MiB output (bf16 4096^3: 128.7 / 132.1).
inline int mfma_store_hint(int types, long long M, long long N, long long K, int out_size, int num_cus) {
  const long long tiles = ((M + 255) / 256) * ((N + 255) / 256);
  if (tiles >= 4ll * num_cus && K * mfma_in_size(types) >= 8192) return 3;
  const long long out_bytes = M * N * out_size;
  return out_bytes <= (64ll << 20) ? 1 : 0;
}

// The launcher's own choice for one launch over the whole problem; returns the estimate it was chosen by.
inline double mfma_choose(int types, int M, int N, int K, int layoutA, int layoutB, int num_cus, MfmaCfg* out) {
  if (num_cus <= 0) num_cus = 256;
  const int in_size = mfma_in_size(types);
  const bool a_rows = layoutA == GZ_ROW_MAJOR, b_cols = layoutB == GZ_COL_MAJOR;
  // candidates: 256x256 and 128x128 (on the ring kernel where the types and the layout of A allow it), 256x128, 64x64
  // (a column-major A beside a row-major B goes through the transposing reads like B, not for the 8-bit floats; beside
  // a column-major B the launcher runs the transposed problem where it can, see mfma_transposed_ring)
  const bool f8_types = types == GZ_E4M3E4M3F16 || types == GZ_E5M2E5M2F16;
  const bool a_direct = a_rows || (!b_cols && !f8_types);
  // (fp32: four waves with a row-major A)
  const bool ring_ok = types == GZ_F32F32F32 ? a_rows : a_direct;
  const bool ring128_ok = ring_ok && !f8_types;
  const int cand[4] = {ring_ok ? MFMA_CFG_RING_W4 : MFMA_CFG_256_W4, MFMA_CFG_256x128,
                       ring128_ok ? MFMA_CFG_RING_128 : MFMA_CFG_128, MFMA_CFG_64};
  double best = 0;
  int pick = cand[0];
  for (int i = 0; i < 4; i++) {
    const MfmaCfg& c = kMfmaCfgs[cand[i]];
    const long long tiles = (long long)((M + c.bm - 1) / c.bm) * ((N + c.bn - 1) / c.bn);
    if (i == 3) {
      // 64 x 64 tiles on the register-staged kernel, several work-groups per compute unit: for grids that larger
      // tiles leave mostly empty.  8-bit elements on two waves.
      double cost64 = -1.0;
      if (types == GZ_F32F32F32) {
        // A 128 x 128 tile is 55 us of fp32 products per 1024 of K on one compute unit, whatever the grid.  A
        // sixteenth of a round of 256 x 256 per tile at 0.75 of the larger tiles' rate (us, 64 x 64 / 128 x 128 tiles,
        // cubes, row/row: 256 8.1 / 21.0, 512 13.7 / 37.3, 1024 25.4 / 70.2, 1536 86.0 / 103.4, 2048 149.5 / 136.7).
        const double share = (double)tiles / (16.0 * num_cus);
        cost64 = (0.05 + 1.35 * (share > 1.0 / 16 ? share : 1.0 / 16)) * 2.2;
      } else if (tiles * 5 <= (b_cols || f8_types ? 10LL : 6LL) * num_cus) {
        // 8- and 16-bit types, up to two tiles per compute unit (int8 and 16-bit, 1.2 with a row-major B: 1280^2 x 2048 22.1 / 20.5, with a
        // K-contiguous B 18.5 / 20.0; 1024 x 2048 x 4096, two per compute unit, 30.1 / 33.5; 1536^2 x 2048, 2.25,
        // 22.1 / 19.9): a tile costs 1.3 + 0.49 us per slab against the
        // 16 + 1.45 of a round of 256 x 256 (us, 64 x 64 / 128 x 128 ring, bf16 -> f32 cubes, row/col: 256 4.7 / 6.3,
        // 512 5.2 / 7.6, 768 7.5 / 10.6, 1024 9.1 / 12.4, 1280 12.5 / 14.5, 1536 18.8 / 16.6; row/row 1024
        // 10.5 / 12.8, 1280 14.8 / 14.9; fp16 the same).
        const double nslab = (double)K * in_size / MFMA_SLAB_BYTES, t = (double)tiles / num_cus;
        cost64 = (1.3 + 0.49 * nslab) / (16.0 + 1.45 * nslab) * (t <= 1.0 ? 0.8 + 0.2 * t : 1.0 + 0.35 * (t - 1.0));
      }
      if (cost64 >= 0 && cost64 < best) {
        best = cost64;
        pick = cand[i];
      }
      continue;
    }
    const long long rounds = (tiles + num_cus - 1) / num_cus;
    // whole tiles: every candidate has a direct-to-LDS kernel; ragged M or N: the 256x256 ones only
    const int cls = mfma_shape_class(c, in_size, M, N, K, layoutA, layoutB);
    const bool direct = (types == GZ_F32F32F32 ? a_rows && (i == 0 || i == 2) : a_direct) &&
                        (cls == MFMA_SHAPE_WHOLE || (cls == MFMA_SHAPE_RAGGED_MN && i == 0));
    // (128 x 128 beyond four rounds: each further round costs a little more, 6144^2 x 6144 = 9 rounds measured
    // 478 us against 457 for three rounds of 256 x 256)
    // (256 x 128 up to one round where every tile has to run on the register-staged kernel - a ragged K, unaligned
    // lines -: 0.62.  1000 x 8000 x 4000 row/row, 252 tiles against
    // 504 of 128 x 128, us: bf16 76 / 82, int8 46 / 50, fp16 79 / 86; 8000 x 1000 x 4096 e4m3 47 / 50)
    double shape_cost = i == 0 ? (double)rounds : i == 1 ? (tiles <= num_cus && cls == MFMA_SHAPE_GENERAL ? 0.62 : 0.75 * rounds)
                                     : 0.40 + 0.27 * rounds + 0.035 * (rounds > 4 ? rounds - 4 : 0);
    const bool f32 = types == GZ_F32F32F32;
    // The register-staged kernel has no second launch for a last round that is mostly empty, but such a round costs
    // less than a whole one: the busy compute units have more of the chip's power and of their L2 (partial rounds of
    // 256 x 256 tiles measured at 0.73 - 0.85 of a whole one for a quarter to three quarters of the compute units).
    // (bf16 6000 x 6000 x 3000, 576 tiles: 261 us against 299 on 128 x 128 tiles, which the whole third round hid.)
    // The ring kernel, persistent past one round, the same way (5120^2 x 4096, 400 tiles: 1.74 of the 4096^2 launch;
    // 6144^2, 576 tiles: 2.69); a grid below one round costs it 0.8 of a round whatever its size (2048^2 0.82,
    // 3072^2 0.83).
    if (i == 0 && !f32) {
      const long long full = tiles / num_cus, rem = tiles % num_cus;
      const double frac = (double)rem / num_cus;
      shape_cost = (double)full + (rem ? 0.65 + 0.25 * frac : 0.0);
      // (the ring kernel: 0.72 of a round up to half a round of tiles, rising to a whole one - 4352 x 4096, 16 tiles
      // left, 0.76; 6144^2, 64, 0.69; 5120^2, 144, 0.74; 5632^2, 228, 0.99)
      if (direct && rem) shape_cost = (double)full + 0.72 + (frac > 0.5 ? 0.56 * (frac - 0.5) : 0.0);
      // below one round (on eight waves, which such a grid gets): 0.77 up to half a round of tiles, rising to a
      // whole one (bf16 K = 4096, us: 81 tiles 74, 128 75, 144 78, 160 80, 192 88 against 97 for 256)
      // (the 8-bit floats 0.81: e4m3 M x 4096 x 4096, 16 ... 128 tiles 40.2 - 40.8 us against 51 for 256)
      if (direct && full == 0) shape_cost = (f8_types ? 0.81 : 0.77) + (frac > 0.5 ? 0.46 * (frac - 0.5) : 0.0);
    }
    // fp32 is bound by its matrix rate at every tile size, so a smaller tile costs what its share of the products
    // costs: 256 x 128 half a round per round of its own, 128 x 128 its tiles over four per compute unit (measured,
    // in rounds of 256 x 256, 128 x 128 / 256 x 128: 6000 x 6000 x 3000 2.56 / 2.69 against 3.19; 3000 x 3000 x 1000
    // 0.79 / 1.03 against 1; 5000^3 1.99 / 2.13 against 2.13; 4096 x 4096 x 4000 1.13 / 1.02 against 1).
    // 128 x 128 tiles on the ring kernel, two work-groups per compute unit: a "double round" of up to 2 x CUs tiles
    // costs 0.36 + 0.15 tiles / CUs of a round of 256 x 256 tiles (bf16 -> f32 cubes, us: 1024 13.5, 1536 21.8, 2048
    // 27.8, 2560 39.0, 3072 74.7 against rounds of 34, 44, 55, 65, 76); the register-staged kernel of the same tile,
    // which the launcher keeps for a K-contiguous B while every work-group has a compute unit to itself, within 0.04
    // of that.
    if (i == 2 && direct && ring128_ok && types != GZ_F32F32F32) {
      const long long full2 = tiles / (2LL * num_cus), rem2 = tiles % (2LL * num_cus);
      shape_cost = 0.66 * full2 + (rem2 ? 0.36 + 0.15 * (double)rem2 / num_cus : 0.0);
    }
    // 128 x 128 tiles on the register-staged kernel (ragged M / N, K-contiguous B), up to three rounds: measured in
    // rounds of 256 x 256, bf16 K = 4096 - 324 tiles 0.70, 504 0.81, 512 0.80, 576 1.09, 640 1.11, 768 1.19 (the line
    // below said 0.99 for the first three and 1.27 for the others, and 2300^2 x 4096 ran 256 x 256 tiles in 82 us
    // instead of these in 67)
    // The 8-bit floats' 128 x 128 tiles (their own direct-to-LDS kernel; no ring instance).  Measured in rounds of
    // 256 x 256 tiles, M x 4096 x 4096 and x 2048, e4m3 - K-contiguous B, one work-group per compute unit at a time:
    // 64 tiles 0.36 / 0.40, 256 0.43 / 0.45, 384 0.65 / 0.66, 512 0.73 / 0.72, 768 1.05 / 1.00, 1024 1.36 / 1.31;
    // row-major B, two at a time: 64 0.59 / 0.58, 256 0.63 / 0.61, 512 0.70 / 0.70, 768 1.26 / 1.23, 1024 1.36 / 1.34.
    bool f8_rowb_fitted = false;
    if (i == 2 && direct && f8_types) {
      if (b_cols) {
        shape_cost = tiles <= num_cus ? 0.36 + 0.07 * (double)tiles / num_cus
                                      : 0.12 + 0.31 * rounds + 0.035 * (rounds > 4 ? rounds - 4 : 0);
      } else {
        const long long full2 = tiles / (2LL * num_cus), rem2 = tiles % (2LL * num_cus);
        shape_cost = 0.68 * full2 + (rem2 ? 0.58 + 0.12 * (double)rem2 / (2.0 * num_cus) : 0.0) + 0.05 * (full2 > 2 ? full2 - 2 : 0);
        f8_rowb_fitted = true;
      }
    }
    bool fitted128 = false;
    if (i == 2 && !direct && !f32 && tiles <= 3LL * num_cus) {
      shape_cost = tiles <= 2LL * num_cus ? 0.50 + 0.30 * (double)tiles / (2.0 * num_cus)
                                          : 1.06 + 0.13 * (double)(tiles - 2LL * num_cus) / num_cus;
      // Against a grid of 256 x 256 tiles below one round these start and end faster and cost more per slab (512
      // tiles against 128 of 256 x 256, ragged, bf16, us: K = 2048 41.5 / 45.8, K = 4096 75.0 / 74.9 - lines of
      // 8 + 1.03 per slab and 16.7 + 0.91 per slab); the figures above are those of K = 4096.  (Not with a row-major
      // B, where the smaller tile's transposing reads take the gain back: K = 2048 47.3 / 44.5.)
      if (tiles <= 2LL * num_cus && b_cols) {
        const double nslab = (double)K * in_size / MFMA_SLAB_BYTES;
        double kf = (8.0 + 1.03 * nslab) / (16.7 + 0.91 * nslab) / 0.987;
        shape_cost *= kf < 0.88 ? 0.88 : kf > 1.06 ? 1.06 : kf;
        // (and 0.94 of that since the ragged epilogue no longer waits for its own stores: 504 - 512 tiles against
        // 128 of 256 x 256, K = 4096, us: 8000 x 1000 75.9 / 78.2, 2000 x 4000 73.2 / 74.7; K = 2048 38.3 / 40.8)
        shape_cost *= 0.94;
      }
      fitted128 = true;
    }
    // (256 x 128 at 0.55 per round of its own: 2560^3, 200 tiles, 313 us against 286 on 400 tiles of 128 x 128 on the
    // ring kernel and 568 for a round of 256 x 256)
    if (f32 && i == 1) shape_cost = 0.55 * rounds;
    // (a grid of fewer 128 x 128 tiles than compute units still takes a whole tile's time)
    if (f32 && i == 2) shape_cost = 0.10 + 1.15 * (tiles > num_cus ? (double)tiles / (4.0 * num_cus) : 0.25);
    // row-major B: the compiler-scheduled kernels of the smaller tiles lose more to the transposing reads
    // (the ring kernel takes a row-major B through the transposing reads at no cost to speak of, on either tile)
    const double rowb = (direct && !b_cols) ? (i == 0 ? 1.0 : i == 1 ? 1.12 : ring128_ok || f8_rowb_fitted ? 1.0 : 1.15) : 1.0;
    // What the register-staged kernel costs over a direct-to-LDS one on the same tile (4096 x 4096 x 4000 against
    // 4096^3, us: bf16 256 x 256 on eight waves 121 / 100, 128 x 128 155 against an estimated 150; int8 73 / 58 and
    // 98 / 87; fp8, four waves, 81 / 52 and 92 / 90).  On 128 x 128 tiles it grows with the rounds beyond four (twice
    // the operand bytes per product through the L2: bf16 6000 x 6000 x 3000, nine rounds, 299 us against 237 by the
    // plain estimate; 5000^3, seven, 352 / 307).  The four waves of the 8-bit floats have a large fixed part per tile
    // (epilogue, first slabs: 8000 x 8000 x 1000 46 us a round, 4096 x 4096 x 4000 81), hence the term in 1 / K
    // (8000 x 8000 x 1000, us, 256 x 256 / 256 x 128 / 128 x 128: 181 / 219 / 154).
    // fp32: 2.2 for every kernel (its round against a round of the 16-bit types; it only weighs the splits), a little
    // less for the hand-scheduled kernel on the 256 x 256 tile.
    const bool f8 = types == GZ_E4M3E4M3F16 || types == GZ_E5M2E5M2F16;
    const double staged = f32 ? 2.2 : i == 2 ? 1.05 + 0.05 * (rounds > 4 ? rounds - 4 : 0)
                                    : f8 ? 1.3 + 1000.0 / (double)(K > 0 ? K : 1) : 1.2;
    const double cost = f32 ? shape_cost * (direct ? 0.95 * 2.2 : 2.2)
                            : shape_cost * rowb * (direct || fitted128 ? 1.0 : staged);
    if (i == 0 || cost < best) {
      best = cost;
      pick = cand[i];
    }
  }
  *out = kMfmaCfgs[pick];
  if (pick == MFMA_CFG_64 && in_size == 1) *out = kMfmaCfg64Int8;
  // (The register-staged kernel of the 128 x 128 tile was kept for a K-contiguous B on grids of up to 5/8 of the compute
  // units.  Interleaved runs of the two, int8 / fp16 / bf16 -> bf16 squares 512 ... 1536 at K = 1024 ... 8192: the ring
  // kernel level or 1 - 4 % ahead on all of them but 1536^2 x 8192, 16-bit, 81 against 74 us; the rule is gone.)
  if (pick == MFMA_CFG_RING_W4) {
    // Waves per 256 x 256 tile on the ring kernel.
    const long long tiles = (long long)((M + 255) / 256) * ((N + 255) / 256);
    const bool f8 = types == GZ_E4M3E4M3F16 || types == GZ_E5M2E5M2F16;
    bool eight = false;
    if (types == GZ_F32F32F32) {
      eight = false;   // one instance: four waves
    } else if (f8) {
      // 8-bit floats: eight waves up to three rounds of tiles (their 16-bit epilogue has more stores in flight),
      // four beyond.  e4m3, us, four / eight waves, row/row: 4096^3 56.2 / 53.3, 5120^3 122.8 / 115.7, 6144^3
      // 221.5 / 213.0, 4096^2 x 8192 99.6 / 99.0, 8192^3 404.9 / 419.4; row/col 4096^3 53.8 / 50.9, 8192^3
      // 386.5 / 401.4.  (A row-major B: eight waves at every size, see below.)
      eight = !(tiles >= 4LL * num_cus && b_cols);
    } else {
      // int8 and the 16-bit types: an estimate of the launch on four and on eight waves, in us per round of tiles,
      // a fixed part (first copies, epilogue) and a part per K slab.  Eight waves (two per SIMD, 128 x 64 per wave)
      // start and end a tile faster - a 16-bit output most of all: its epilogue is bound by the number of its stores,
      // and two waves per SIMD keep more of them in flight - but read a quarter more LDS bytes per product, which
      // costs per slab with a K-contiguous B (where four waves issue one copy per eight MFMAs and nothing else) and
      // nothing with a row-major B (whose transposing reads, two per fragment, four waves have to fit between their
      // MFMAs).  Fitted to squares 3072 ... 8192, K = 1024 and 4096, us, four / eight waves -
      // bf16 -> f32 row/col: 3072^2 29.8 / 30.3, 80.3 / 89.1; 4096^2 34.2 / 36.4, 96.6 / 103.4; 5120^2 59.3 / 57.0,
      // 167.8 / 170.4; 6144^2 92.4 / 88.5, 259.6 / 261.8; 8192^2 147.4 / 156.1, 388.9 / 421.2;
      // bf16 -> bf16 row/col: 3072^2 31.2 / 29.6, 81.7 / 88.7; 4096^2 33.9 / 31.5, 96.1 / 98.0; 5120^2 60.4 / 54.0,
      // 167.2 / 167.9; 8192^2 133.8 / 129.3, 376.7 / 393.0; row/row 4096^2 34.9 / 31.5, 101.3 / 97.9; 5120^2
      // 63.3 / 54.8, 174.2 / 168.2; 8192^2 143.3 / 136.1, 387.7 / 385.5;
      // bf16 -> f32 row/row: 4096^2 35.1 / 36.5, 101.5 / 101.2; 5120^2 61.7 / 58.7, 175.8 / 173.6; 8192^2
      // 154.2 / 155.9, 398.2 / 415.6; int8 row/col 4096^2 24.1 / 25.3, 55.2 / 58.6; 5120^2 42.1 / 38.4, 94.4 / 94.2;
      // 8192^2 106.0 / 106.2, 231.6 / 248.9.
      // (a column-major A beside a row-major B: both operands through the transposing reads, two per fragment, which
      // four waves cannot fit between their MFMAs - eight at every size: bf16 4096^3 101 / 98 us, 5120^2 x 4096
      // 188 / 174, 7168^2 x 4096 377 / 356, 8000 x 1000 x 4096 94 / 76)
      const bool out16 = types == GZ_BF16BF16BF16 || types == GZ_F16F16F16;
      const double nslab = (double)K * in_size / MFMA_SLAB_BYTES;
      const bool under_a_round = tiles < num_cus, whole_rounds = tiles % num_cus == 0;
      const double slope4 = b_cols ? 1.30 : 1.38;
      double slope8 = slope4 * (b_cols ? (under_a_round ? 1.17 : 1.07) : (under_a_round ? 1.11 : 0.985));
      if (tiles >= 3LL * num_cus) slope8 *= 1.05;   // past three rounds four waves pull ahead (8192^2 x 4096 above)
      const double fixed4 = out16 ? 13.6 : 13.2;
      const double fixed8 = out16 ? 9.6 : whole_rounds ? 14.1 : 10.5;   // compute units left empty: more of the power and of the L2 for the busy ones
      // Below one round: eight.  With half the compute units idle the busy ones are not held by power, the slopes are
      // the same and eight waves' fixed part is 8 us lower (about 140 tiles, us, four / eight waves, K = 2048 and 4096:
      // row/col 54.3 / 46.0, 86.7 / 78.2; row/row 55.3 / 46.0, 89.3 / 77.6; whole tiles, 3072^2: 79.1 / 76.6, 80.5 / 73.7).
      // (Ragged M and N follow the same rule: us, four / eight waves, row/col then row/row - bf16 -> f32 4095 x 4096 x
      // 1024 34.1 / 37.2, 34.8 / 35.6; 8000 x 8192 x 2048 218.6 / 240.9, 222.6 / 242.0; fp16 4095 x 4096 x 1024
      // 34.3 / 33.8, 35.1 / 32.4; 8000 x 8192 x 2048 219.5 / 230.7, 231.6 / 226.6; int8 8000 x 8000 x 8192 379 / 414,
      // 402 / 420.)
      // (Below one round with a ragged M or N, a K-contiguous B and a 32-bit output the estimate decides as well (a
      // row-major B stays on eight: 2000 x 4000 x 4096 75.2 / 71.0): us, four / eight waves,
      // bf16 -> f32 row/col 3000^2 x 4096 70.8 / 76.4, 4000 x 3000 x 2048 48.1 / 53.9, 8000 x 1000 x 4096 76.3 / 79.3,
      // int8 3000 x 4096 x 2048 28.6 / 31.1; a 16-bit output stays on eight, bf16 -> bf16 3000 x 4096 x 2048 47.4 / 45.3.)
      const bool ragged = M % 256 != 0 || N % 256 != 0;
      eight = !a_rows || (under_a_round && (!ragged || out16 || !b_cols)) || fixed8 + slope8 * nslab < fixed4 + slope4 * nslab;
    }
    if (eight) *out = kMfmaCfgs[MFMA_CFG_RING_W8];
  }
  return best;
}

inline bool mfma_resolve(int types, int M, int N, int K, int layoutA, int layoutB, int variant, int num_cus,
                         MfmaCfg* out) {
  if (variant < 0 || variant > kNumMfmaCfgs) return false;
  if (variant > 0) {
    *out = kMfmaCfgs[variant - 1];
    // (8-bit elements: on two waves)
    if (out->bm == 64 && mfma_in_size(types) == 1) *out = kMfmaCfg64Int8;
    return true;
  }
  (void)mfma_choose(types, M, N, K, layoutA, layoutB, num_cus, out);
  return true;
}

// The launcher's choice once the class of the launch is known.  A 256 x 256 tile that has to run on the register-staged
// kernel (ragged K, unaligned operands) wants eight waves for 8-bit integers and 16-bit floats with a row-major A
// (4096 x 4096 x 4000, us, four / eight waves: int8 96 / 82 and 103 / 84 with a row-major B, bf16 161 / 133 and
// 180 / 149) and four for the 8-bit floats, whose eight-wave instance does not fit its registers (105 / 206).
inline void mfma_adjust_general(int types, int cls, int layoutA, int layoutB, MfmaCfg* c) {
  // (whole tiles of a column-major A are in the "whole" class and still run on that kernel; they gain as well:
  // 4096^3, int8 84 / 77, bf16 135 / 124 and 144 / 128 with a row-major B)
  const bool f8 = types == GZ_E4M3E4M3F16 || types == GZ_E5M2E5M2F16;
  const bool a_staged = layoutA != GZ_ROW_MAJOR && (layoutB != GZ_ROW_MAJOR || f8 || types == GZ_F32F32F32);
  const bool staged = cls == MFMA_SHAPE_GENERAL || a_staged;
  if (!staged || c->bm != 256 || c->bn != 256) return;
  if (f8) *c = kMfmaCfgs[MFMA_CFG_256_W4];
  else if (types != GZ_F32F32F32) *c = kMfmaCfgs[MFMA_CFG_256_W8];
  else *c = kMfmaCfgs[MFMA_CFG_256_W4];
}

// Ragged last round.  When the 256x256 tiles of a problem fill some rounds of the compute units and then leave a
// last round mostly empty (6144 x 6144: 576 tiles = 2.25 rounds of 256), one launch pays for a whole round more.
// With a row-major A the rows of the problem can be cut in two launches instead, since row ranges of A, C and D
// are packed matrices themselves: the first covers as many tile rows as fit whole rounds, with 256x256 tiles, the
// second the remaining rows with whatever tile the estimate above prefers for them (usually 128x128, which spreads
// the leftover over all compute units).  Taken when the summed estimate is at least 3 % below the single launch.
struct MfmaSplit {
  int rows_main;      // rows of the first launch (a multiple of 256), 0 = no split
  MfmaCfg main, tail;
};
inline bool mfma_resolve_split(int types, int M, int N, int K, int layoutA, int layoutB, int num_cus, MfmaSplit* out,
                               double* estimate = nullptr) {
  out->rows_main = 0;
  if (num_cus <= 0) num_cus = 256;
  if (layoutA != GZ_ROW_MAJOR || M < 512 || N <= 0 || K <= 0) return false;
  // a second launch costs its fixed part (first copies, epilogue, the gap) whatever K is; below about 24 slabs a
  // round is too short to win that back (us, two launches / one launch on eight waves, K = 512, 1024, 4096 -
  // bf16 4608^2 40.8 / 38.3, 57.2 / 56.9, 159.1 / 170.3; int8 40.3 / 38.2 at K = 1024, 92.6 / 94.1 at 4096)
  if ((long long)K * mfma_in_size(types) < 24 * MFMA_SLAB_BYTES) return false;
  MfmaCfg single;
  const double cost_single = mfma_choose(types, M, N, K, layoutA, layoutB, num_cus, &single);
  const long long tiles_n = (N + 255) / 256, tiles_m = (M + 255) / 256;
  const long long full = tiles_m * tiles_n / num_cus * num_cus;   // tiles in whole rounds
  if (full == 0 || full == tiles_m * tiles_n) return false;
  // Only where few tiles remain: the ring kernel's persistent launch carries a larger remainder better than a second
  // launch does (5120^2 x 4096, 144 of 400 tiles remain, us, one launch / two: bf16 167.7 / 170.3, row-major B
  // 170.2 / 176.9, int8 95.2 / 99.5; with 16 remaining the cut wins: 4352 x 4096^2 row/row 149 / 141, 7168^2 355 / 338).
  if (tiles_m * tiles_n - full > num_cus / 4) return false;
  const long long tile_rows = full / tiles_n;                     // tile rows that fit them
  if (tile_rows <= 0 || tile_rows * 256 >= M) return false;
  const int rows_main = (int)(tile_rows * 256);
  MfmaCfg main_cfg, tail_cfg;
  double cost_main = mfma_choose(types, rows_main, N, K, layoutA, layoutB, num_cus, &main_cfg);
  if (main_cfg.bm != 256 || main_cfg.bn != 256) return false;
  // only where the first launch runs a direct-to-LDS kernel, whose speed the estimate knows well
  if (mfma_shape_class(main_cfg, mfma_in_size(types), rows_main, N, K, layoutA, layoutB) == MFMA_SHAPE_GENERAL) return false;
  const double cost_tail = mfma_choose(types, M - rows_main, N, K, layoutA, layoutB, num_cus, &tail_cfg);
  if (cost_main + cost_tail > 0.97 * cost_single) return false;
  if (estimate) *estimate = cost_main + cost_tail;
  out->rows_main = rows_main;
  out->main = main_cfg;
  out->tail = tail_cfg;
  return true;
}

// A few columns past a multiple of 256.  N = 4097 puts one column of data into a seventeenth column of 256-wide
// tiles, each of which costs what a whole tile costs, and where the whole ones just fill the compute units that is
// a round of its own (fp16 4096 x 4097 x 1024, K-contiguous B: 80 us against 42 for N = 4096).  Cut off instead:
// the first launch covers the columns up to the multiple of 256, the second the few that remain: up to
// MFMA_STRIP_MAX_COLS of them as dot products, one wave per row (mfma_strip_kernel), more as an M x r problem on small
// tiles (about 0.45 of a round of whole tiles: 15-18 us at K = 1024, 44-52 at K = 4096).  Both
// address C, D and a row-major B with the row pitch of the whole matrices (ldb / ldd of the kernel arguments), which
// the register-staged tile kernel and the epilogues take; with a K-contiguous B the first launch keeps the
// hand-scheduled kernel.  Taken when the estimate is at least 3 % below the single launch.
constexpr int MFMA_STRIP_MAX_COLS = 8;   // up to here the cut-off columns run as dot products (mfma_strip_kernel), not as tiles
struct MfmaColSplit {
  int cols_main;      // columns of the first launch (a multiple of 256), 0 = no split
  MfmaCfg main, tail;
  bool strip;         // the cut-off columns run as dot products (mfma_strip_kernel), not as tiles
};
inline bool mfma_transposed_ring(int types, int M, int N, int K, int layoutA, int layoutB, int variant, int num_cus,
                                 MfmaCfg* out, MfmaSplit* split);
inline bool mfma_resolve_colsplit(int types, int M, int N, int K, int layoutA, int layoutB, int num_cus, MfmaColSplit* out,
                                  double* estimate = nullptr) {
  out->cols_main = 0;
  if (num_cus <= 0) num_cus = 256;
  const int r = N % 256;
  if (N < 512 || r == 0 || r > 64 || M <= 0 || K <= 0) return false;
  MfmaCfg single;
  double cost_single = mfma_choose(types, M, N, K, layoutA, layoutB, num_cus, &single);
  const int cols_main = N - r;
  MfmaCfg main_cfg, tail_cfg;
  double cost_main = mfma_choose(types, M, cols_main, K, layoutA, layoutB, num_cus, &main_cfg);
  // (column-major A and B: what the ring kernel on the transposed problem costs, where it takes the whole problem
  // and where it takes the first launch)
  if (MfmaCfg t; mfma_transposed_ring(types, M, N, K, layoutA, layoutB, 0, num_cus, &t, nullptr))
    cost_single = mfma_choose(types, N, M, K, GZ_ROW_MAJOR, GZ_ROW_MAJOR, num_cus, &t);
  if (MfmaCfg t; mfma_transposed_ring(types, M, cols_main, K, layoutA, layoutB, 0, num_cus, &t, nullptr))
    cost_main = mfma_choose(types, cols_main, M, K, GZ_ROW_MAJOR, GZ_ROW_MAJOR, num_cus, &t);
  // the first launch keeps the ring kernel on a 256 x 256 tile where the layouts allow it and the rows of a
  // row-major B, which keep the pitch of the whole matrix, are whole 16-byte pieces
  const int cls = mfma_shape_class(main_cfg, mfma_in_size(types), M, cols_main, K, layoutA, layoutB);
  const bool f8_types = types == GZ_E4M3E4M3F16 || types == GZ_E5M2E5M2F16;
  const bool layouts_ok = layoutA == GZ_ROW_MAJOR || (layoutB == GZ_ROW_MAJOR && !f8_types);
  const bool direct_before = layouts_ok && types != GZ_F32F32F32 &&
                             (cls == MFMA_SHAPE_WHOLE || (cls == MFMA_SHAPE_RAGGED_MN && main_cfg.bm == 256 && main_cfg.bn == 256));
  const bool direct_after = direct_before && main_cfg.bm == 256 && main_cfg.bn == 256 &&
                            (layoutB == GZ_COL_MAJOR || ((long long)N * mfma_in_size(types)) % 16 == 0);
  if (direct_before && !direct_after) cost_main *= types == GZ_F32F32F32 ? 2.2 : mfma_in_size(types) == 2 ? 1.2 : 1.5;
  // on the register-staged kernel eight waves carry a 256 x 256 tile of 16-bit elements better than four
  // (fp16 4095 x 4097 x 1023, row-major B: 119 us against 158)
  if (!direct_after && main_cfg.bm == 256 && main_cfg.bn == 256 && mfma_in_size(types) == 2) main_cfg = kMfmaCfgs[MFMA_CFG_256_W8];
  tail_cfg = kMfmaCfgs[MFMA_CFG_128];   // 128 x 128: the strip in as many work-groups as it has row blocks
  // What the cut-off columns cost depends on K, the rounds above do not say it: in us, the dot products
  // 3 + (M / 4096) (K bytes / 2048) (4 + 1.8 r) (one column of 4095 x 1023 fp16: 11 us; eight of 4096 x 4096: 75),
  // the same strip on 128 x 128 tiles 5 + 11.5 (M / 4096) (K bytes / 2048) (15-18 us at K = 1024, 44-52 at 4096),
  // against a round of 256 x 256 tiles at 16 + 1.45 per 128 bytes of K.  The cheaper of the two is taken, so a
  // long K sends even a few columns to the tiles (4096 x 4104 x 4096: 51 instead of 75 us beside a main launch
  // of 108).
  const double k_units = (double)K * mfma_in_size(types) / 2048.0, m_units = (double)M / 4096.0;
  const double round_us = 16.0 + 1.45 * ((double)K * mfma_in_size(types) / 128.0);
  // (a column-major A is read by the dot products in pieces of rows, a line of memory per k: 2.5 x - col/col
  // 4096 x 4099 x 4096 took 200 us with the strip against 172 in one launch)
  const double strip_us = (3.0 + m_units * k_units * (4.0 + 1.8 * r)) * (layoutA == GZ_ROW_MAJOR ? 1.0 : 2.5),
               tiles_us = 5.0 + 11.5 * m_units * k_units;
  out->strip = r <= MFMA_STRIP_MAX_COLS && strip_us <= tiles_us;
  const double cost_tail = (out->strip ? strip_us : tiles_us) / round_us;
  if (cost_main + cost_tail > 0.97 * cost_single) return false;
  if (estimate) *estimate = cost_main + cost_tail;
  out->cols_main = cols_main;
  out->main = main_cfg;
  out->tail = tail_cfg;
  return true;
}

// Both cuts may apply to one problem (4096 x 4097: a 17th tile column that also spills into a second round): the one
// with the lower estimate is taken.  Returns 0 (one launch), 1 (rows) or 2 (columns).
inline int mfma_resolve_cut(int types, int M, int N, int K, int layoutA, int layoutB, int num_cus, MfmaSplit* rows,
                            MfmaColSplit* cols) {
  double est_rows = 0, est_cols = 0;
  const bool by_rows = mfma_resolve_split(types, M, N, K, layoutA, layoutB, num_cus, rows, &est_rows);
  const bool by_cols = mfma_resolve_colsplit(types, M, N, K, layoutA, layoutB, num_cus, cols, &est_cols);
  if (by_rows && by_cols) return est_cols <= est_rows ? 2 : 1;
  return by_rows ? 1 : by_cols ? 2 : 0;
}

// Stream-K.  When the 256 x 256 tiles of a problem fill some whole rounds of the compute units and then leave R more
// (5120^2: 400 tiles = one round of 256 and 144), a plain launch pays a whole round for those R.  Here the R tiles'
// slabs, R * (K / slab) of them in one sequence, are dealt to `blocks` further work-groups of the same launch in equal
// contiguous runs; a run covers the end of one tile or that and the start of the next, leaves its sums in a slot of
// a workspace, and a second small launch adds each tile's pieces in a fixed order and writes D (the reference has the
// same tail: its persistent grid of min(#SM, tiles) work-groups, nvidia/kernel_functors/bf16_mma_gemm.cuh:42-48).
// Only on the kernel with the 16x16 instructions: row-major A, either layout of B, whole K slabs, 16-byte aligned rows.
struct StreamKPlan {
  int dp_tiles, sk_tiles, blocks, q, rem;   // see struct StreamK of the kernel
  int slots;                                // workspace slots of 256 x 256 accumulators
  MfmaCfg cfg;                              // tile configuration (the ring kernel on four or eight waves)
  double estimate_us;
};
constexpr long long MFMA_STREAMK_SLOT_BYTES = 256ll * 256 * 4;
// forced: an explicit stream-K variant: taken wherever it can run; otherwise only where the estimate says so
inline bool mfma_plan_streamk(int types, int M, int N, int K, int layoutA, int layoutB, int num_cus, bool forced,
                              const MfmaCfg* forced_cfg, StreamKPlan* out) {
  if (num_cus <= 0) num_cus = 256;
  const int in_size = mfma_in_size(types);
  if (!(types == GZ_S8S8S32 || in_size == 2) || layoutA != GZ_ROW_MAJOR) return false;
  MfmaCfg cfg;
  double single_rounds = mfma_choose(types, M, N, K, layoutA, layoutB, num_cus, &cfg);
  if (forced) cfg = kMfmaCfgs[forced_cfg->waves_n == 4 ? MFMA_CFG_RING_W8 : MFMA_CFG_RING_W4];
  else if (cfg.id != MFMA_VARIANT_RING_W4 && cfg.id != MFMA_VARIANT_RING_W8) {
    // a smaller tile was preferred for the whole problem (few tiles): stream-K still competes, on the 256 x 256 tile
    cfg = kMfmaCfgs[in_size == 2 ? MFMA_CFG_RING_W8 : MFMA_CFG_RING_W4];
  }
  // Below one round of tiles every work-group is a piece whose sums leave as fp32 whatever the output type, so the
  // eight waves' faster 16-bit epilogue does not apply and four waves' cheaper main loop does (bf16 -> f32, us, four /
  // eight waves: 1024^2 x 8192 43.6 / 46.1, 1280^2 x 8192 56.4 / 61.0, 2048^2 x 8192 72.6 / 77.5, x 16384
  // 113.8 / 124.2).
  if (!forced && (long long)((M + 255) / 256) * ((N + 255) / 256) < num_cus) cfg = kMfmaCfgs[MFMA_CFG_RING_W4];
  if (mfma_shape_class(cfg, in_size, M, N, K, layoutA, layoutB) == MFMA_SHAPE_GENERAL) return false;
  const int nslab = K / (MFMA_SLAB_BYTES / in_size);
  const long long tiles = (long long)((M + 255) / 256) * ((N + 255) / 256);
  const int R = (int)(tiles % num_cus);
  const long long full = tiles - R;
  if (R == 0 || full > 0x7fffffff / 2) return false;
  const int min_slabs = forced ? 2 : 8;
  long long blocks = (long long)R * nslab / min_slabs;
  if (blocks > num_cus) blocks = num_cus;
  blocks -= blocks % 8;
  if (blocks <= R) return false;   // every run shorter than a tile: q < nslab
  const long long total = (long long)R * nslab;
  out->dp_tiles = (int)full;
  out->sk_tiles = R;
  out->blocks = (int)blocks;
  out->q = (int)(total / blocks);
  out->rem = (int)(total % blocks);
  out->slots = (int)blocks + R - 1;
  out->cfg = cfg;
  // Estimate, us.  A round of 256 x 256 tiles: a fixed part (first copies, epilogue, the write of a round's D)
  // and 1.45 us per slab (bf16 4096^3: 23.2 us per 1024 of K; int8 moves the same bytes per slab).  A stream-K
  // work-group runs q + 1 slabs; what the decomposition costs beyond that - the pieces' stores into the workspace,
  // which all work-groups issue at about the same moment, and the second launch, which reads every slot once and
  // writes the R tiles - was fitted to the launches below as 14 + 0.058 slots + 0.25 R (30 us at R = 16 / 271
  // slots, 47 at 68 / 323, 50 at 105 / 360, 72 at 144 / 399).
  // Measured, bf16 -> f32, us, plain launch / stream-K / what the launcher takes (hipBLASLt): where few tiles
  // remain or the grid is small and K long it wins - 4352 x 4096 x 4096 (16 of 272 tiles remain) 166 / 137 / 129
  // (134), 7168^2 x 4096 (16 of 784) 366 / 339 / 336 (395), 2048^2 x 8192 (64 tiles) 135 / 78 / 76 (69),
  // 1024^2 x 16384 (16 tiles) 261 / 55 / 54 (62) - and where most of a round remains it loses: the partial sums
  // are then 100 MiB, and a last round that is half empty costs less than half a round more on a part whose clock
  // follows power: 5120^3 (144 of 400 remain) 221 / 264 / 221 (224), int8 117 / 155 / 117 (132), 4864^2 x 4096
  // 174 / 189 / 172 with the rows cut in two launches (162), 4608^3 192 / 188 / 180 the same way (168).
  const int out_size = (types == GZ_S8S8S32 || types == GZ_BF16BF16F32) ? 4 : 2;
  const double slab_us = 1.45, fixed_us = out_size == 4 ? 16.0 : 11.0;
  const double round_us = fixed_us + nslab * slab_us;
  const double overhead_us = 14.0 + 0.058 * out->slots + 0.25 * R;
  out->estimate_us = (double)(full / num_cus) * round_us + (out->q + 1) * slab_us + overhead_us;
  if (forced) return true;
  // No whole round (a grid smaller than the device): every work-group streams its own K range of its own tile, so
  // nothing is shared through the L2s and the operands come from memory once per tile; against 128 x 128 tiles,
  // one or two per compute unit, that pays only for a long K and few tiles.  Measured, us, stream-K / 128 x 128
  // tiles, bf16 K = 2048, 4096, 8192, 16384: 512^2 (4 tiles) 19.5 / 19.7, 23.0 / 34.3, 23.5 / 63.6, 31.0 / 123;
  // 1024^2 (16) 23.3 / 19.9, 27.1 / 34.8, 40.9 / 65.9, 54.8 / 125; 1280^2 (25) - , 33.9 / 34.9, 54.7 / 65.0,
  // 86.7 / 125; 1536^2 (36) - , 48.3 / 37.6, 67.1 / 66.1, 116 / 158; 1792^2 (49) - , 52.3 / 39.1, 84.5 / 71.6,
  // 149 / 158; 2048^2 (64) - , - , 76.0 / 79.7, 126 / 167; 2560^2 (100) at 8192 147 / 112 (256 x 128 tiles);
  // int8 (slabs of 128 K) 768^2 at K = 4096 31.3 / 18.2, 8192 24.6 / 31.4; 1536^2 at 8192 49.1 / 34.1,
  // 16384 68.3 / 62.5.  In slabs: at least 48 and at least four per tile of the grid.
  // Where the runs are whole fractions of a tile - every work-group one piece, none that ends one tile and begins the
  // next with a second 256 KiB store - two slabs per tile of the grid are enough (2048^2 x 8192: 64 tiles in quarters,
  // 72.6 us against 82.6 on 128 x 128 tiles; 1792^2 x 8192, 49 tiles in runs of 24.5 slabs: 85.5 against 79.7).
  const bool whole_fractions = out->rem == 0 && nslab % out->q == 0;
  const int per_tile = whole_fractions ? 2 : 4;
  if (full == 0 && nslab < (per_tile * R > 48 ? per_tile * R : 48)) return false;
  // past whole rounds only where few tiles remain: between an eighth and most of a round the estimates of the
  // alternatives are not sharp enough to tell (4608^3: 180 us with the rows cut in two launches, 188 here)
  // (two whole rounds and a quarter: 6144^2 x 4096, 64 of 576 tiles remain, 248 us against 268 in one plain launch)
  if (full > 0 && R > (full >= 2LL * num_cus ? num_cus / 4 : num_cus / 8)) return false;
  // what the launcher would do otherwise, in the same unit (its estimates count rounds of 256 x 256 tiles)
  MfmaSplit sp;
  MfmaColSplit cs;
  double est_rows = 0, est_cols = 0, best = single_rounds;
  if (mfma_resolve_split(types, M, N, K, layoutA, layoutB, num_cus, &sp, &est_rows) && est_rows < best) best = est_rows;
  if (mfma_resolve_colsplit(types, M, N, K, layoutA, layoutB, num_cus, &cs, &est_cols) && est_cols < best) best = est_cols;
  return out->estimate_us < 0.99 * best * round_us;
}

// Work-groups of a launch of whole tiles on the ring kernel: past one round of the compute units the kernel is
// persistent, one work-group per compute unit walking tiles b, b + grid, ... (the order in which the hardware deals
// work-groups out anyway) and asking for its next tile's first slab before it stores the current one.  (Variants 9
// and 10 launch one work-group per tile instead, for comparisons.)
inline long long mfma_persistent_grid(long long tiles, int num_cus) {
  if (num_cus <= 0) num_cus = 256;
  return tiles > num_cus ? num_cus : tiles;
}

// Shape class of a launch.  Beyond the extents, the direct-to-LDS kernels and the unpredicated register-staged one
// need 16-byte aligned operands and lines (leading dimensions that are whole 16-byte pieces) and address a tile's
// lines with 32-bit byte offsets from its first; the whole-tile epilogue stores 16 bytes per lane, so the rows of C and
// D must be whole 16-byte pieces as well, or the launch takes the epilogue of the ragged kernels.
// A column-major A with a column-major B is the transposed problem D^T = B^T A^T: B^T is N x K with K contiguous, a
// row-major first operand, and A^T is K x M, a row-major second operand.  The ring kernel runs that pair (it takes the
// MFMA operands in the other order and writes the real, row-major D), and does so 10-15 % faster than the
// register-staged kernel runs the problem as given.  Taken where ONE launch of the ring kernel covers the transposed
// problem - the launcher's own choice for it is that kernel and neither a cut nor stream-K, or the caller names a
// variant of the ring kernel - and its tiles are whole (or ragged in M / N on the 256 x 256 tile).  Fills `out` with
// the configuration in terms of the transposed problem (bm along N, bn along M).
// `split`, if given: a row cut of the transposed problem (columns of the real one) where the launcher would make one and
// both parts run the ring kernel; rows_main = 0 otherwise.
inline bool mfma_transposed_ring(int types, int M, int N, int K, int layoutA, int layoutB, int variant, int num_cus,
                                 MfmaCfg* out, MfmaSplit* split = nullptr) {
  if (split) split->rows_main = 0;
  if (layoutA != GZ_COL_MAJOR || layoutB != GZ_COL_MAJOR || M <= 0 || N <= 0 || K <= 0) return false;
  if (variant < 0 || variant > kNumMfmaCfgs) return false;
  if (variant > 0) {
    *out = kMfmaCfgs[variant - 1];
  } else {
    (void)mfma_choose(types, N, M, K, GZ_ROW_MAJOR, GZ_ROW_MAJOR, num_cus, out);
    MfmaSplit sp;
    const int in_size = mfma_in_size(types);
    auto whole = [&](const MfmaCfg& c, int rows) {
      return c.ring != 0 && !c.stream_k && mfma_shape_class(c, in_size, rows, M, K, GZ_ROW_MAJOR, GZ_ROW_MAJOR) == MFMA_SHAPE_WHOLE;
    };
    // (the remaining rows on the ring kernel's small tile where the estimate took a tile that kernel does not have)
    if (split && types != GZ_E4M3E4M3F16 && types != GZ_E5M2E5M2F16 &&
        mfma_resolve_split(types, N, M, K, GZ_ROW_MAJOR, GZ_ROW_MAJOR, num_cus, &sp) && whole(sp.main, sp.rows_main) &&
        whole(sp.tail.ring ? sp.tail : (sp.tail = kMfmaCfgs[MFMA_CFG_RING_128]), N - sp.rows_main)) {
      *split = sp;
      *out = sp.main;
    }
  }
  if (out->ring == 0 || out->stream_k) return false;
  const bool f8 = types == GZ_E4M3E4M3F16 || types == GZ_E5M2E5M2F16;
  if (f8 && out->bm != 256) return false;   // the 8-bit floats have the 256 x 256 tile only on that kernel
  // (and their slab schedule wants eight row blocks per wave, which the eight-wave tile laid out the other way round
  // does not have: four waves)
  if ((f8 || types == GZ_F32F32F32) && out->waves_m * out->waves_n == 8) *out = kMfmaCfgs[out->id - 2];
  if (types == GZ_F32F32F32 && out->bm != 256 && out->id != kMfmaCfgs[MFMA_CFG_RING_128].id) return false;
  const int cls = mfma_shape_class(*out, mfma_in_size(types), N, M, K, GZ_ROW_MAJOR, GZ_ROW_MAJOR);
  return cls == MFMA_SHAPE_WHOLE || (cls == MFMA_SHAPE_RAGGED_MN && out->bm == 256);
}

inline int mfma_launch_class(const MfmaCfg& c, int in_size, int out_size, int M, int N, int K, int layoutA, int layoutB,
                             const void* A, const void* B, const void* C, const void* D, long long lda, long long ldb,
                             long long ldc, long long ldd) {
  const uintptr_t bits = (uintptr_t)A | (uintptr_t)B | (uintptr_t)C | (uintptr_t)D;
  if (bits & 15u) return MFMA_SHAPE_GENERAL;
  if ((lda * in_size) % 16 || (ldb * in_size) % 16) return MFMA_SHAPE_GENERAL;
  if (lda * in_size * 256 >= (1LL << 32) || ldb * in_size * 256 >= (1LL << 32)) return MFMA_SHAPE_GENERAL;
  int cls = mfma_shape_class(c, in_size, M, N, K, layoutA, layoutB);
  if (cls == MFMA_SHAPE_WHOLE && ((ldd * out_size) % 16 || (C && (ldc * out_size) % 16))) {
    const int epv = 16 / in_size;
    const bool a_ok = layoutA == GZ_ROW_MAJOR || (layoutB == GZ_ROW_MAJOR && M % epv == 0);
    cls = (a_ok && (layoutB == GZ_COL_MAJOR || N % epv == 0)) ? MFMA_SHAPE_RAGGED_MN : MFMA_SHAPE_GENERAL;
  }
  return cls;
}

}  // namespace gz
