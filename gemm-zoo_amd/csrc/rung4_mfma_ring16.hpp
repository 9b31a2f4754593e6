// MFMA rung, whole-line ring of five LDS buffers with the 16x16 matrix instructions.
//
// Data movement: every copy asks the L2 for whole 128-byte lines (8 rows x 128 bytes of K per instruction), so a K
// slab (128 bytes of K per row) is cut by ROWS into two copy groups; a group fills one of five 32 KiB buffers (all of
// the LDS), one barrier per slab.  Arithmetic:
//     v_mfma_f32_16x16x32_{bf16,f16}   v_mfma_i32_16x16x64_i8   v_mfma_f32_16x16x128_f8f6f4
// rather than the 32x32 forms.  A 16x16 instruction sums 64 bytes of K per row inside the matrix pipe before it
// touches the accumulators, a 32x32 one 32 bytes, so the same product costs half the accumulator reads and writes -
// and this part runs against its power limit: an MFMA-only loop on N(0,1) bf16 operands sustains 2100-2130 TFLOPS
// with the 16x16x32 instruction against 1835-1855 with 32x32x16 (at 2.06 against 1.79 GHz), 1920-1970 against
// 1710-1735 with the fragment reads of a 256x256 tile interleaved.
//
// A K step is 64 bytes of K per row: a 128-byte slab has two of them, each with (WM / 16) x (WN / 16) MFMAs of
// 16 cycles and WM / 16 + WN / 16 fragment reads.  Per slab j (groups 2j, 2j+1 in buffers (2j) % 5, (2j+1) % 5):
//   K step 0 : MFMAs on set 0; requests the fragments of (j, 1) into set 1; issues copy group 2j+4 (A rows, then
//              B rows) into buffer (2j+4) % 5, which slab j-1 left at its barrier
//   barrier  : lgkmcnt(0) - every read of slab j has returned, its two buffers are free afterwards;
//              vmcnt(n)   - this wave's copies of groups 2j+2 and 2j+3 have landed (the n of group 2j+4 may fly)
//   K step 1 : MFMAs on set 1; requests the fragments of (j+1, 0) into set 0; issues all of copy group 2j+5 into
//              buffer (2j) % 5
// A step's fragment reads follow every RDE-th MFMA of its first three quarters, so that they have returned when the
// next step asks for them; its copies are spread evenly over the whole step, one every NMMA / NCP MFMAs: issued as
// one run behind the reads they cost 1-5 % more (bf16 4096^3 100.5 -> 99.3 us, int8 8192^3 434.5 -> 418.0 on four
// waves; eight waves at K = 8192: 213.9 -> 198.1).
// What the loop costs is power, not waiting: the copies of a bf16 4096^3 launch alone take 60 us (17.5 TB/s into the
// compute units), its MFMAs alone 63, both together 77 at a lower clock (bench/probe_operand_stream.cpp), this loop
// with its fragment reads and barriers 83.  Timing-only builds of this kernel say the same: no barrier and no wait at
// all 99.2 against 100.5 us for the launch, the copies as plain register loads with no LDS write 106.5 against 106.8,
// all copies from one slab (always L2 hits) 96.5, no copies in the main loop 84.2; a different first slab per tile
// (so that tiles that share rows do not ask for them at the same moment) lost 1-4 %; copies switched off by a zero
// lane mask for three of four waves in turn 140 us (exec = 0 is not free).
//
// Fragments: lane l supplies row l % 16 and the 16 bytes of K at piece 4 s + q(l) of K step s, q(l) the two bits of
// l / 16 swapped (see below); tile row
// r = 16 G + 8 p + i lives in the buffer of group parity p at G * 1024 + i * 128, piece c at slot c ^ i ^ p, so
// the sixteen rows of sixteen consecutive lanes fall into the sixteen four-bank groups.  The B fragment is the
// instruction's first operand: a lane ends up with four consecutive columns of one row of D,
//     acc[i][j][e] = D(row0 + 16 i + l % 16, col0 + 16 j + 4 (l / 16) + e).
//
// K a multiple of the slab (128 bytes); either layout of A and of B (template parameters below); whole tiles, or
// (RAGGED) any M and N with 16-byte aligned lines.
#pragma once

namespace gz {

template <int TYPES> using AccVec4 = AccVec4Of<TYPES>;

template <int TYPES>
__device__ __forceinline__ void asm_mfma16(typename AccVec4<TYPES>::type& c, const u32x4_t& first, const u32x4_t& second) {
  if constexpr (TYPES == GZ_S8S8S32)
    asm volatile("v_mfma_i32_16x16x64_i8 %0, %1, %2, %0" : "+a"(c) : "v"(first), "v"(second));
  else if constexpr (TYPES == GZ_F16F16F16)
    asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(c) : "v"(first), "v"(second));
  else
    asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(c) : "v"(first), "v"(second));
}
// fp32: v_mfma_f32_16x16x4_f32 takes one value per lane and operand, lane l row l % 16 and k = l / 16.  A 16-byte
// fragment holds four consecutive k of the lane's row: four instructions, each on one register of the two fragments
// (instruction S sums k = 4 (l / 16) + S over the four lane groups; A and B agree on that, which is all it needs).
template <int S> __device__ __forceinline__ void asm_mfma16_f32(f32x4_t& c, uint32_t first, uint32_t second) {
  asm volatile("v_mfma_f32_16x16x4_f32 %0, %1, %2, %0" : "+a"(c) : "v"(first), "v"(second));
}
template <int TYPES> __device__ __forceinline__ void asm_touch_acc4(typename AccVec4<TYPES>::type& c) {
  asm volatile("" : "+a"(c));
}
// 8-bit floats: v_mfma_f32_16x16x128_f8f6f4 takes 32 bytes per lane and operand, here the 16-byte fragments of both
// K steps of a slab side by side (which k a lane's bytes stand for is the same on A and B, and that is all a dot
// product needs).  cbsz / blgp select the format of the two operands: 0 e4m3, 1 e5m2.
template <int TYPES>
__device__ __forceinline__ void asm_mfma16_f8(typename AccVec4<TYPES>::type& c, const u32x8_t& f, const u32x8_t& s) {
  if constexpr (TYPES == GZ_E5M2E5M2F16)
    asm volatile("v_mfma_f32_16x16x128_f8f6f4 %0, %1, %2, %0 cbsz:1 blgp:1" : "+a"(c) : "v"(f), "v"(s));
  else
    asm volatile("v_mfma_f32_16x16x128_f8f6f4 %0, %1, %2, %0" : "+a"(c) : "v"(f), "v"(s));
}
__device__ __forceinline__ u32x8_t join8(const u32x4_t& lo, const u32x4_t& hi) {
  return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
}
__device__ __forceinline__ u32x4_t join4(const u32x2_t& lo, const u32x2_t& hi) {
  return __builtin_shufflevector(lo, hi, 0, 1, 2, 3);
}
__device__ __forceinline__ void asm_touch_v4(u32x4_t& a, u32x4_t& b) { asm volatile("" : "+v"(a), "+v"(b)); }
// A transposing read at addr ^ XOR.  The 16-column blocks of a wave's part of a row-major B lie at addresses that
// differ from the first block's in two or three bits only (see b_addr), so one address register per buffer and an
// exclusive-or in front of the read replace a register per (buffer, block): 5 instead of 40 with four waves.
template <int ES, int OFF, int XOR> __device__ __forceinline__ void asm_ds_read_tr_x(u32x2_t& dst, uint32_t addr) {
  if constexpr (XOR == 0) {
    asm_ds_read_tr<ES, OFF>(dst, addr);
  } else {
    uint32_t t;
    if constexpr (ES == 2)
      asm volatile("v_xor_b32 %1, %3, %2\n\tds_read_b64_tr_b16 %0, %1 offset:%4" : "=v"(dst), "=&v"(t) : "v"(addr), "i"(XOR), "i"(OFF));
    else
      asm volatile("v_xor_b32 %1, %3, %2\n\tds_read_b64_tr_b8 %0, %1 offset:%4" : "=v"(dst), "=&v"(t) : "v"(addr), "i"(XOR), "i"(OFF));
  }
}
// Two 4-byte values, OFF0 and OFF1 times 256 bytes past addr ^ XOR (fp32 fragments of a row-major B: two K rows).
template <int OFF0, int OFF1, int XOR> __device__ __forceinline__ void asm_ds_read32x2_x(u32x2_t& dst, uint32_t addr) {
  static_assert(OFF0 >= 0 && OFF0 < 256 && OFF1 >= 0 && OFF1 < 256, "8-bit offsets in units of 64 dwords");
  if constexpr (XOR == 0) {
    asm volatile("ds_read2st64_b32 %0, %1 offset0:%2 offset1:%3" : "=v"(dst) : "v"(addr), "i"(OFF0), "i"(OFF1));
  } else {
    uint32_t t;
    asm volatile("v_xor_b32 %1, %3, %2\n\tds_read2st64_b32 %0, %1 offset0:%4 offset1:%5"
                 : "=v"(dst), "=&v"(t) : "v"(addr), "i"(XOR), "i"(OFF0), "i"(OFF1));
  }
}
__device__ __forceinline__ void asm_touch_v2(u32x2_t& a, u32x2_t& b, u32x2_t& c, u32x2_t& d) {
  asm volatile("" : "+v"(a), "+v"(b), "+v"(c), "+v"(d));
}

// Stream-K launch (STREAMK = true).  The tiles of the problem, in the order of their logical ids, are the `dp_tiles`
// that fill whole rounds of the compute units, one work-group each as in a plain launch, and then `sk_tiles` more whose
// slabs - sk_tiles * (K / slab) of them, taken as one sequence tile after tile - are dealt to `blocks` further
// work-groups in equal contiguous runs (q or q + 1 slabs each, q less than a tile's slabs): a run is the end of one
// tile, or that and the beginning of the next.  Every such piece leaves its 256 x 256 sums, as accumulated, in its
// own slot of the workspace (slot = block + tile: unique, at most blocks + sk_tiles - 1 of them);
// streamk_fixup_kernel then adds a tile's pieces in the order of their blocks - a fixed order, so the result does not
// depend on timing - and applies alpha, beta and the output rounding.  Nothing waits for anything inside a kernel.
struct StreamK {
  int dp_tiles, sk_tiles, blocks, q, rem;
  void* ws;
};
__host__ __device__ inline int streamk_first_slab(const StreamK& sk, int b) { return b * sk.q + (b < sk.rem ? b : sk.rem); }
__host__ __device__ inline int streamk_block_of_slab(const StreamK& sk, int it) {
  const int big = sk.rem * (sk.q + 1);
  return it < big ? it / (sk.q + 1) : sk.rem + (it - big) / sk.q;
}
constexpr size_t STREAMK_SLOT_ELEMS = 256 * 256;

// Row-major B: where 16-byte piece p of K row r (within its copy group) sits in that row of the LDS buffer.  A
// transposing read takes, per 16 lanes, a block of 4 (16-bit) or 8 (int8) K rows, and the four lane groups of a
// fragment take blocks 8 (16) rows apart: the first term spreads the rows of a block over the banks, the second
// the two blocks that one half of the wave reads in the same cycle.
// (Rows of 128 bytes - int8 with a 128-column tile - hold eight pieces, and consecutive rows already lie in different
// halves of the 64 banks: the row's lowest bit stays out of the swizzle, which then fits three bits.)
// fp32 has no transposing read: a lane takes one value per K row (two rows per ds_read2st64_b32), sixteen lanes
// sixteen consecutive columns of it (64 bytes) and the four lane groups K rows four apart, which the swizzle sends
// 64 bytes apart.
template <int ES, int ROW_BYTES> __host__ __device__ constexpr int ring16_row_swizzle(int r) {
  static_assert(ROW_BYTES >= 256 || (ES == 1 && ROW_BYTES == 128), "a K row of at least sixteen pieces, or eight of int8");
  return ES == 4 ? (((r >> 2) & 3) << 2) : ES == 2 ? (((r & 3) << 2) ^ (((r >> 3) & 1) << 1))
                 : ROW_BYTES >= 256 ? (((r & 7) << 1) ^ ((r >> 4) & 1)) : ((((r >> 1) & 3) << 1) ^ ((r >> 4) & 1));
}

// SWAP: the launch is the transposed problem D^T = B^T A^T of a column-major A with a column-major B.  B^T (N x K,
// K contiguous) is this kernel's first operand and A^T (K x M, M contiguous) its second, a "row-major B": g.A, g.B,
// g.M, g.N, g.lda and g.ldb come swapped by the launcher, g.C / g.D / g.ldc / g.ldd are those of the real row-major
// output.  The MFMAs take their operands in the other order, so that a lane still ends up with four consecutive
// columns of one row of the real D, and the epilogue walks the accumulator blocks transposed; nothing else changes.
// A_KC = false: a column-major A (K rows of M contiguous elements) beside a row-major B.  A then takes the route of a
// row-major B: whole K rows per copy, a K step per copy group, fragments through the transposing LDS reads.
template <int TYPES, int BM, int BN, int WAVES_M, int WAVES_N, bool RAGGED = false, bool STREAMK = false, bool B_KC = true,
          bool SWAP = false, bool A_KC = true>
// (second launch bound: waves per SIMD the registers must leave room for - the 128 x 128 tile, whose five buffers are
// half the LDS, runs two work-groups per compute unit)
__global__ void __launch_bounds__(WAVES_M* WAVES_N * 64, (BM == 128 && BN == 128) ? 2 : (WAVES_M * WAVES_N) / 4)
    mfma_ring16_kernel(GemmArgs<TYPES> g, int tiles_m, int tiles_n, StreamK sk) {
  using T = Traits<TYPES>;
  using in_t = typename T::in_t;
  using acc_v = typename AccVec4<TYPES>::type;
  constexpr int NW = WAVES_M * WAVES_N;
  constexpr int ES = (int)sizeof(in_t);
  constexpr int LINE = 128;           // K bytes per row and slab
  constexpr int SK = LINE / ES;       // K elements per slab
  constexpr int NST = 5;              // LDS buffers, one copy group each
  constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;
  constexpr int FM = WM / 16, FN = WN / 16;
  constexpr bool F32 = TYPES == GZ_F32F32F32;
  constexpr int SUB = F32 ? 4 : 1;    // matrix instructions per 16 x 16 block and K step
  // fp32 with a row-major B (and not the transposed problem): four consecutive COLUMNS per lane, see b4 below
  constexpr bool B4 = F32 && !B_KC && !SWAP;
  constexpr int NRD_A = A_KC ? FM : 2 * FM, NRD_B = (B_KC || B4) ? FN : 2 * FN;
  constexpr int NMMA = FM * FN, NRD = NRD_A + NRD_B;   // MFMAs and LDS reads per K step
  constexpr int EPV = 16 / ES;
  constexpr int HK = 64 / ES;         // K rows of a row-major B per copy group: one K step
  constexpr bool F8 = is_fp8(TYPES);
  static_assert(!STREAMK || (A_KC && !SWAP), "stream-K with a row-major A (either layout of B)");
  static_assert(!SWAP || !B_KC, "the transposed problem of two column-major operands has a row-major second operand");
  static_assert(!(F8 && STREAMK), "stream-K for int8 and the 16-bit types");
  static_assert(A_KC || (!B_KC && !SWAP && !STREAMK && !F8), "a column-major A with a row-major B, int8 and the 16-bit types");
  constexpr int A_BYTES = BM / 2 * LINE, B_BYTES = BN / 2 * LINE;
  constexpr int STAGE_BYTES = A_BYTES + B_BYTES;
  constexpr int A_PW = BM / 16 / NW, B_PW = BN / 16 / NW;  // 1 KiB copies (8 rows) per wave and group
  constexpr int NCP = A_PW + B_PW;
  static_assert(!F32 || (NW == 4 && A_KC && !STREAMK), "fp32: four waves, row-major A");
  static_assert((BM == 256 && BN == 256) || (BM == 128 && BN == 128 && NW == 4 && !F8 && !STREAMK),
                "the 256 x 256 tile, or the 128 x 128 tile on four waves for int8 and the 16-bit types");
  static_assert(BM % (16 * NW) == 0 && BN % (16 * NW) == 0, "tile rows must divide over the waves");
  static_assert(A_PW <= 8 && B_PW <= 8 && A_PW % 2 == 0 && B_PW % 2 == 0, "a copy group must fit the immediate offset range");
  static_assert(NCP == 8 || NCP == 4, "the vmcnt immediates below are written out for 8 or 4 copies per wave and group");

  extern __shared__ __attribute__((aligned(1024))) char lds[];
  const uint32_t lds_base = (uint32_t)(uintptr_t)lds;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave % WAVES_M, wn = wave / WAVES_M;
  const int K = g.K;
  const int nslab_all = K / SK;
  // the run of slabs of this work-group: [it, it_end) of the stream-K sequence (STREAMK, past the whole tiles)
  int it = 0, it_end = 0, sk_block = 0;
  if constexpr (STREAMK) {
    static_assert(BM == 256 && BN == 256, "a workspace slot is one 256 x 256 tile");
    if ((int)blockIdx.x >= sk.dp_tiles) {
      // every XCD a contiguous share of the sequence (work-groups are dealt to the XCDs round-robin)
      const int bp = (int)blockIdx.x - sk.dp_tiles;
      sk_block = sk.blocks % 8 == 0 ? (bp % 8) * (sk.blocks / 8) + bp / 8 : bp;
      it = streamk_first_slab(sk, sk_block);
      it_end = streamk_first_slab(sk, sk_block + 1);
    }
  }
  // A launch of fewer work-groups than tiles (no stream-K) is a persistent one: work-group b takes
  // tiles b, b + gridDim.x, ... in the order the hardware would have dealt them, and asks for the first slab (copy
  // groups 0 and 1) of its next tile before it stores the current one, so that it arrives during the epilogue
  // instead of after a new work-group's start.
  constexpr bool PERSISTENT = !STREAMK;
  int bid = (int)blockIdx.x;
  bool prefetched = false;   // groups 0 and 1 of this pass's tile are already on their way
  for (;;) {
  int tm, tn, slab0 = 0, nslab_seg = nslab_all;
  bool partial = false;
  int slot = 0;
  if constexpr (STREAMK) {
    if ((int)blockIdx.x < sk.dp_tiles) {
      tile_of_lid(lid_of_block(blockIdx.x, sk.dp_tiles), tiles_m, tiles_n, tm, tn);
    } else {
      const int tt = it / nslab_all;
      slab0 = it - tt * nslab_all;
      nslab_seg = min(nslab_all - slab0, it_end - it);
      partial = true;
      slot = sk_block + tt;
      tile_of_lid(sk.dp_tiles + tt, tiles_m, tiles_n, tm, tn);
    }
  } else {
    tile_of_block(bid, tiles_m, tiles_n, tm, tn);
  }
  const int m0 = tm * BM, n0 = tn * BN;
  const int nc = 2 * nslab_seg;  // copy groups
  const size_t k_byte0 = (size_t)slab0 * LINE;   // first K byte of this run within a row

  // ---- copy addressing: lane -> (row ci of the 8 rows of a copy, LDS slot cs) ----
  // A copy is ONE instruction of the main loop, with nothing scalar around it.  Its source address has three parts:
  // a scalar base that every copy of the operand in a K step shares (the tile's first row at the K offset of the
  // slab that is being fetched; a_cp / b_cp below, advanced once per slab or K step), a per-lane offset kept in a
  // register per (parity, copy of the group) and computed once per tile - which 16 rows, which parity, the lane's
  // row and piece - and the immediate.  The immediate also moves the LDS address (that is what it is for: the copies
  // of a group step through LDS with it, under one M0), so it is taken off the per-lane offset again; COPY_BIAS keeps
  // that difference non-negative and is taken off the scalar base.  (Before: one scalar base per copy, computed in
  // the loop with four to six scalar instructions, and a compare and a branch around every copy for the groups past
  // the end of K - seven to ten instructions per copy between two MFMAs, where a wave that is alone on its SIMD issues one
  // instruction every four cycles and an MFMA leaves room for three.)
  constexpr uint32_t COPY_BIAS = 4096;
  const int ci = lane >> 3, cs = lane & 7;
  const int N = g.N;
  const size_t LDA = (size_t)g.lda * ES, LDB = (size_t)g.ldb * ES;   // bytes between the lines of A and of B
  // row-major B: group c carries K rows [HK c, HK c + HK) of B, BN elements each; a copy moves KRC whole K rows, the
  // lane at LDS position (row, slot) fetching the piece that belongs there (see ring16_row_swizzle)
  constexpr int KRC = 1024 / (BN * ES), LPR = 64 / KRC;
  static_assert(B_KC || (KRC * BN * ES == 1024 && NW * B_PW * KRC == HK), "whole K rows per copy, a K step per group");
  constexpr int KRC_A = 1024 / (BM * ES), LPR_A = 64 / KRC_A;
  static_assert(A_KC || (KRC_A * BM * ES == 1024 && NW * A_PW * KRC_A == HK), "whole K rows per copy, a K step per group");
  uint32_t voff_a[A_KC ? 2 : 1][A_PW], voff_b[B_KC ? 2 : 1][B_PW];
  const size_t a_group_step = A_KC ? 0 : (size_t)HK * LDA, b_group_step = B_KC ? 0 : (size_t)HK * LDB;
  // (the offsets of the tile whose first row and column are m_first, n_first: they differ between tiles only where
  // RAGGED clamps rows or columns)
  auto set_copy_offsets = [&](int m_first, int n_first) {
#pragma unroll
    for (int par = 0; par < 2; par++) {
      if constexpr (A_KC) {
#pragma unroll
        for (int t = 0; t < A_PW; t++) {
          // RAGGED: rows past the end are fetched from the last row (an output depends on its own row of A and column
          // of B only, and those past the end are not stored)
          int r = 16 * (wave * A_PW + t) + 8 * par + ci;
          if constexpr (RAGGED) r = min(m_first + r, g.M - 1) - m_first;
          voff_a[par][t] = (uint32_t)((size_t)r * LDA + (size_t)((cs ^ ci ^ par) * 16)) + COPY_BIAS - (uint32_t)((t - A_PW / 2) * 1024);
        }
      }
      if constexpr (B_KC) {
#pragma unroll
        for (int t = 0; t < B_PW; t++) {
          int r = 16 * (wave * B_PW + t) + 8 * par + ci;
          if constexpr (RAGGED) r = min(n_first + r, N - 1) - n_first;
          voff_b[par][t] = (uint32_t)((size_t)r * LDB + (size_t)((cs ^ ci ^ par) * 16)) + COPY_BIAS - (uint32_t)((t - B_PW / 2) * 1024);
        }
      }
    }
    if constexpr (!A_KC) {
      const int last_piece = (g.M - m_first) / EPV - 1;   // RAGGED: M is a multiple of EPV on this path, m_first < M
#pragma unroll
      for (int t = 0; t < A_PW; t++) {
        const int kr = (wave * A_PW + t) * KRC_A + lane / LPR_A;   // K row within the group
        int piece = (lane % LPR_A) ^ ring16_row_swizzle<ES, BM * ES>(kr);
        if constexpr (RAGGED) piece = min(piece, last_piece);      // rows past the end: the last piece (not stored)
        voff_a[0][t] = (uint32_t)((size_t)kr * LDA + (size_t)(piece * EPV) * ES) + COPY_BIAS - (uint32_t)((t - A_PW / 2) * 1024);
      }
    }
    if constexpr (!B_KC) {
      const int last_piece = (N - n_first) / EPV - 1;   // RAGGED: N is a multiple of EPV on this path, n_first < N
#pragma unroll
      for (int t = 0; t < B_PW; t++) {
        const int kr = (wave * B_PW + t) * KRC + lane / LPR;   // K row within the group
        int piece = (lane % LPR) ^ ring16_row_swizzle<ES, BN * ES>(kr);
        if constexpr (RAGGED) piece = min(piece, last_piece);  // columns past the end: the last piece (not stored)
        voff_b[0][t] = (uint32_t)((size_t)kr * LDB + (size_t)(piece * EPV) * ES) + COPY_BIAS - (uint32_t)((t - B_PW / 2) * 1024);
      }
    }
  };
  set_copy_offsets(m0, n0);
  // scalar bases of a tile: its first row of A (first column of a K-contiguous B) at the first K byte of this run; a
  // row-major B's first K row of the run at the tile's first column
  auto a_base_of = [&](int m_first) -> const char* {
    if constexpr (A_KC) return reinterpret_cast<const char*>(g.A) + (size_t)m_first * LDA + k_byte0 - COPY_BIAS;
    else return reinterpret_cast<const char*>(g.A) + (size_t)(2 * slab0) * HK * LDA + (size_t)m_first * ES - COPY_BIAS;
  };
  auto b_base_of = [&](int n_first) -> const char* {
    if constexpr (B_KC) return reinterpret_cast<const char*>(g.B) + (size_t)n_first * LDB + k_byte0 - COPY_BIAS;
    else return reinterpret_cast<const char*>(g.B) + (size_t)(2 * slab0) * HK * LDB + (size_t)n_first * ES - COPY_BIAS;
  };
  // where copy group C of a tile starts, from the tile's bases
  auto a_group = [&](const char* a_tile, int c) -> const char* {
    if constexpr (A_KC) return a_tile + (size_t)(c >> 1) * LINE;
    else return a_tile + (size_t)c * a_group_step;
  };
  auto b_group = [&](const char* b_tile, int c) -> const char* {
    if constexpr (B_KC) return b_tile + (size_t)(c >> 1) * LINE;
    else return b_tile + (size_t)c * b_group_step;
  };
  const uint32_t m0_a = lds_base + (wave * A_PW) * 1024 + (A_PW / 2) * 1024;
  const uint32_t m0_b = lds_base + A_BYTES + (wave * B_PW) * 1024 + (B_PW / 2) * 1024;
  auto copy_a_begin = [&](int st) { asm_set_m0(m0_a + st * STAGE_BYTES); };
  auto copy_b_begin = [&](int st) { asm_set_m0(m0_b + st * STAGE_BYTES); };
  auto copy_a = [&](auto t_c, auto p_c, const char* src) {
    constexpr int Tn = decltype(t_c)::value, P = decltype(p_c)::value, OFF = (Tn - A_PW / 2) * 1024;
    asm_copy16<OFF>(voff_a[A_KC ? P : 0][Tn], src);
  };
  auto copy_b = [&](auto t_c, auto p_c, const char* src) {
    constexpr int Tn = decltype(t_c)::value, P = decltype(p_c)::value, OFF = (Tn - B_PW / 2) * 1024;
    asm_copy16<OFF>(voff_b[B_KC ? P : 0][Tn], src);
  };

  // ---- fragment addressing: one LDS byte address per (slab position in the ring, K step) ----
  // Which quarter of a K step (8 consecutive k of 16-bit types, 16 of int8) a lane group holds is free as long as A
  // and B agree.  Lanes l and l + 32 go through the LDS in the same cycle: with the natural order (quarter l / 16)
  // they would read pieces two apart of the same rows, which the swizzle sends to the same banks for rows i and
  // i ^ 2 (SQ_LDS_BANK_CONFLICT: 48 % of the LDS-active cycles, though no time: 97.6 against 98.1 us); with the two bits
  // of l / 16 swapped they read neighbouring pieces, which never meet (counter 0 on four waves).
  const int fp = (lane >> 3) & 1, fi = lane & 7;
  const int quarter = ((lane >> 5) & 1) | (((lane >> 4) & 1) << 1);
  uint32_t a_addr[NST][A_KC ? 2 : 1], b_addr[NST][B_KC ? 2 : 1];   // transposing reads: per buffer, the wave's first 16-wide block
#pragma unroll
  for (int jr = 0; jr < NST; jr++) {
    const int buf = (2 * jr + fp) % NST;
#pragma unroll
    for (int ks = 0; ks < 2; ks++) {
      const int pos = ((ks * 4 + quarter) ^ fi ^ fp) * 16;
      if constexpr (A_KC) a_addr[jr][ks] = lds_base + buf * STAGE_BYTES + (wm * WM / 16) * 1024 + fi * LINE + pos;
      if constexpr (B_KC) b_addr[jr][ks] = lds_base + buf * STAGE_BYTES + A_BYTES + (wn * WN / 16) * 1024 + fi * LINE + pos;
    }
  }
  // Transposing reads of a row-major B (ds_read_b64_tr_b16 / _b8): within 16 lanes, lane i supplies the address of
  // 8 bytes of a block of 4 (8) K rows x 16 columns, row by row, and receives column i: 4 (8) consecutive K values.
  // Lane group l / 16 takes the K rows of its quarter of the step; two reads, 4 (8) rows apart, make one fragment.
  constexpr int TR_LPR = ES == 2 ? 4 : 2;                 // lanes per K row of a block
  constexpr int TR_PITCH = BN * ES;                       // bytes between K rows
  constexpr int TR_R_OFF = (16 / TR_LPR) * TR_PITCH;      // second half of a fragment
  if constexpr (B4) {
    // A 16-byte read of a K row gives a lane four consecutive columns.  Lane group q of read g takes K row 4 q + g
    // (the k that register g of the A fragment stands for), lane c of the group columns 4 c .. 4 c + 3 of a group
    // of 64: register s of the read is then a B fragment for the sixteen columns 4 c + s, and the four
    // instructions on (register g of A, register s of read g) for g = 0 .. 3 sum the sixteen k of the step into
    // accumulator block 4 G + s of column group G.  One read per four MFMAs' worth of B, as with a K-contiguous B;
    // the epilogue knows the column order (BY4).
    static_assert(!B4 || (WN % 64 == 0 && 3 * TR_PITCH + (WN / 64 - 1) * 256 < 65536), "immediate offsets");
    const int krow = quarter * 4;
    const int f = ring16_row_swizzle<ES, BN * ES>(krow);
#pragma unroll
    for (int st = 0; st < NST; st++) {
      const int piece = ((wn * WN) / EPV + (lane & 15)) ^ f;
      b_addr[st][0] = lds_base + st * STAGE_BYTES + A_BYTES + krow * TR_PITCH + piece * 16;
    }
  } else if constexpr (!B_KC && F32) {
    // fp32: lane group q takes K rows 4 q + S (S by the immediate offset), the lane column l % 16 of the block
    static_assert(!F32 || B_KC || (WN % 64 == 0 && (TR_PITCH & (TR_PITCH - 1)) == 0 && STAGE_BYTES % TR_PITCH == 0 &&
                                   A_BYTES % TR_PITCH == 0 && 3 * TR_PITCH < 65536), "block addresses differ by an exclusive-or");
    const int krow = quarter * 4;
    const int f = ring16_row_swizzle<ES, BN * ES>(krow);   // the same for the four rows of a lane group
#pragma unroll
    for (int st = 0; st < NST; st++) {
      const int n_local = wn * WN + (lane & 15);
      const int piece = (n_local / EPV) ^ f;
      b_addr[st][0] = lds_base + st * STAGE_BYTES + A_BYTES + krow * TR_PITCH + piece * 16 + (n_local % EPV) * ES;
    }
  } else if constexpr (!B_KC) {
    static_assert(B_KC || TR_R_OFF < 65536, "immediate offset");
    const int i16 = lane & 15, ti = i16 / TR_LPR;
    const int n_sub = (i16 % TR_LPR) * (8 / ES);
    const int krow = quarter * (2 * 16 / TR_LPR) + ti;
    const int f = ring16_row_swizzle<ES, BN * ES>(krow);           // the same for the second half: its rows differ in bit 2 (3) only
    // Block j of the wave starts 16 j columns further, i.e. 16 j / EPV pieces: j pieces for 8-bit elements, 2 j for
    // 16-bit ones.  Those are bits of the piece number that nothing else of it touches (the wave's first column is
    // a multiple of 64, the lane's column within a block less than 16), the swizzle is an exclusive-or on the piece
    // number, and a row has fewer than TR_PITCH / 16 pieces: so block j's address is block 0's with
    // j * TR_BLOCK_XOR exclusive-ored in.
    static_assert(B_KC || (WN % 64 == 0 && FN * 16 * ES / 16 <= 16 && (TR_PITCH & (TR_PITCH - 1)) == 0 &&
                           STAGE_BYTES % TR_PITCH == 0 && A_BYTES % TR_PITCH == 0), "block addresses differ by an exclusive-or");
#pragma unroll
    for (int st = 0; st < NST; st++) {
      const int n_local = wn * WN + n_sub;
      const int piece = (n_local / EPV) ^ f;
      b_addr[st][0] = lds_base + st * STAGE_BYTES + A_BYTES + krow * TR_PITCH + piece * 16 + (n_local % EPV) * ES;
    }
  }
  constexpr int TR_BLOCK_XOR = 16 * ES;   // 16 columns = 16 ES bytes of a K row: one piece of 8-bit, two of 16-bit elements
  // a column-major A the same way: K rows of BM elements at the start of each buffer
  constexpr int TR_PITCH_A = BM * ES, TR_R_OFF_A = (16 / TR_LPR) * TR_PITCH_A;
  if constexpr (!A_KC) {
    static_assert(A_KC || (WM % 64 == 0 && FM * 16 * ES / 16 <= 16 && (TR_PITCH_A & (TR_PITCH_A - 1)) == 0 &&
                           STAGE_BYTES % TR_PITCH_A == 0 && TR_R_OFF_A < 65536), "block addresses differ by an exclusive-or");
    const int i16 = lane & 15, ti = i16 / TR_LPR;
    const int m_sub = (i16 % TR_LPR) * (8 / ES);
    const int krow = quarter * (2 * 16 / TR_LPR) + ti;
    const int f = ring16_row_swizzle<ES, BM * ES>(krow);
#pragma unroll
    for (int st = 0; st < NST; st++) {
      const int m_local = wm * WM + m_sub;
      const int piece = (m_local / EPV) ^ f;
      a_addr[st][0] = lds_base + st * STAGE_BYTES + krow * TR_PITCH_A + piece * 16 + (m_local % EPV) * ES;
    }
  }

  acc_v acc[FM][FN];
#pragma unroll
  for (int i = 0; i < FM; i++)
#pragma unroll
    for (int j = 0; j < FN; j++)
#pragma unroll
      for (int v = 0; v < 4; v++) acc[i][j][v] = 0;
  static_for<NMMA>([&](auto q_c) {
    constexpr int Q = decltype(q_c)::value;
    asm_touch_acc4<TYPES>(acc[Q / FN][Q % FN]);
  });
  asm volatile("s_nop 7" ::: "memory");
  u32x4_t af[2][FM], bf[2][FN];  // register sets of fragments: one per K step of a slab
  u32x2_t bh[2][B_KC ? 1 : FN][2];  // row-major B: the two halves of a fragment as they come out of the transposing reads
  u32x2_t ah[2][A_KC ? 1 : FM][2];  // column-major A: the same
  u32x2_t bq[2][(F32 && !B_KC && !B4) ? FN : 1][2];   // fp32, transposed problem: a fragment's four values, two K rows per read
  u32x4_t b4[2][B4 ? FN / 4 : 1][4];                  // fp32, row-major B: [column group][read g], four columns each

  // 16 rows of a fragment are one 1 KiB row group
  auto read_one = [&](auto set_c, auto r_c, auto jr_c) {
    constexpr int SET = decltype(set_c)::value, R = decltype(r_c)::value, JR = decltype(jr_c)::value;
    // (transposing reads: K step SET of the slab at ring position JR is copy group 2 JR + SET, whole, in its own buffer)
    if constexpr (R < NRD_A) {
      if constexpr (A_KC) asm_ds_read16<R * 1024>(af[SET][R], a_addr[JR][SET]);
      else {
        constexpr int I = R / 2, HALF = R % 2, ST = (2 * JR + SET) % NST;
        asm_ds_read_tr_x<ES, HALF * TR_R_OFF_A, I * TR_BLOCK_XOR>(ah[SET][I][HALF], a_addr[ST][0]);
      }
    } else if constexpr (B_KC) asm_ds_read16<(R - NRD_A) * 1024>(bf[SET][R - NRD_A], b_addr[JR][SET]);
    else if constexpr (B4) {
      constexpr int G = (R - NRD_A) / 4, RG = (R - NRD_A) % 4, ST = (2 * JR + SET) % NST;
      asm_ds_read16<RG * TR_PITCH + G * 256>(b4[SET][G][RG], b_addr[ST][0]);
    } else if constexpr (F32) {
      constexpr int J = (R - NRD_A) / 2, HALF = (R - NRD_A) % 2, ST = (2 * JR + SET) % NST;
      static_assert(!F32 || B_KC || TR_PITCH % 256 == 0, "K rows whole units of the two-address read apart");
      asm_ds_read32x2_x<2 * HALF * (TR_PITCH / 256), (2 * HALF + 1) * (TR_PITCH / 256), J * TR_BLOCK_XOR>(bq[SET][J][HALF], b_addr[ST][0]);
    } else {
      constexpr int J = (R - NRD_A) / 2, HALF = (R - NRD_A) % 2, ST = (2 * JR + SET) % NST;
      asm_ds_read_tr_x<ES, HALF * TR_R_OFF, J * TR_BLOCK_XOR>(bh[SET][J][HALF], b_addr[ST][0]);
    }
  };

  // One K step: NMMA MFMAs on register set SET, rows of blocks walked back and forth so that consecutive
  // instructions share an operand.  Between them the NRD fragment reads of (ring position RJ, K step SET ^ 1) into
  // the other set, and the copies of a group of parity CP into buffer CST from a_src / b_src: the A rows in the first
  // half, the B rows in the second.  The last two slabs of a run have nothing left to fetch: their copies fetch the
  // run's last slab once more (a_src / b_src stop advancing there), into buffers that nothing reads any more.  A
  // copy that is switched off costs more than one that runs: under an all-zero lane mask it still takes its place in
  // the memory pipeline, and the two writes of exec around it took two of the three issue slots an MFMA leaves -
  // and a second instance of the step without copies made the register allocator give up the accumulators' places
  // across the branches (it spilled 950 - 1800 registers).
  auto kstep = [&](auto set_c, auto rj_c, auto cp_c, auto cst_c, const char* a_src, const char* b_src) {
    constexpr int SET = decltype(set_c)::value, CST = decltype(cst_c)::value;
    // MFMAs per copy: over the whole step (bf16 4096^3, us: copies over the whole step 97.7, over its first half
    // 99.2, all at its start 104.4)
    constexpr int CPE = NMMA * SUB / NCP;
    // MFMAs per read: the reads end with the third quarter of the step (with both operands through the transposing
    // reads on the small tile there are as many reads as MFMAs: one behind each)
    constexpr int RDE = (NMMA * SUB * 3 / 4) / NRD >= 1 ? (NMMA * SUB * 3 / 4) / NRD : 1;
    static_assert(NRD <= NMMA * SUB, "a step's reads fit between its MFMAs");
    asm volatile("s_waitcnt lgkmcnt(0)");
    if constexpr (!B_KC && !F32) {
#pragma unroll
      for (int j = 0; j < FN; j++) {
        asm volatile("" : "+v"(bh[SET][j][0]), "+v"(bh[SET][j][1]));  // after the wait
        bf[SET][j] = u32x4_t{bh[SET][j][0][0], bh[SET][j][0][1], bh[SET][j][1][0], bh[SET][j][1][1]};
      }
    }
    if constexpr (!A_KC) {
#pragma unroll
      for (int i = 0; i < FM; i++) {
        asm volatile("" : "+v"(ah[SET][i][0]), "+v"(ah[SET][i][1]));
        af[SET][i] = u32x4_t{ah[SET][i][0][0], ah[SET][i][0][1], ah[SET][i][1][0], ah[SET][i][1][1]};
      }
    }
    // (fp32: four sweeps over the blocks, one per register of the fragments, so that the four instructions of a block
    // lie NMMA instructions apart and none waits for the one before on the same accumulators)
    static_for<NMMA * SUB>([&](auto q_c) {
      constexpr int Q = decltype(q_c)::value, S = Q / NMMA, QB = Q % NMMA;
      constexpr int I = QB / FN, J = (I & 1) ? FN - 1 - QB % FN : QB % FN;
      if constexpr (F32) {
        if constexpr (B_KC) asm_mfma16_f32<S>(acc[I][J], bf[SET][J][S], af[SET][I][S]);
        else if constexpr (B4) asm_mfma16_f32<S>(acc[I][J], b4[SET][J / 4][S][J % 4], af[SET][I][S]);
        else if constexpr (SWAP) asm_mfma16_f32<S>(acc[I][J], af[SET][I][S], bq[SET][J][S / 2][S % 2]);
        else asm_mfma16_f32<S>(acc[I][J], bq[SET][J][S / 2][S % 2], af[SET][I][S]);
      } else if constexpr (SWAP) asm_mfma16<TYPES>(acc[I][J], af[SET][I], bf[SET][J]);
      else asm_mfma16<TYPES>(acc[I][J], bf[SET][J], af[SET][I]);
      if constexpr (Q % RDE == RDE - 1 && Q / RDE < NRD)
        read_one(std::integral_constant<int, SET ^ 1>{}, std::integral_constant<int, Q / RDE>{}, rj_c);
      constexpr int Tc = Q / CPE;
      if constexpr (Q == 0) copy_a_begin(CST);
      if constexpr (Q == CPE * A_PW) copy_b_begin(CST);
      if constexpr (Q % CPE == CPE / 2) {
        if constexpr (Tc < A_PW) copy_a(std::integral_constant<int, Tc>{}, cp_c, a_src);
        else copy_b(std::integral_constant<int, Tc - A_PW>{}, cp_c, b_src);
      }
    });
  };

  // 8-bit floats.  One MFMA covers the whole slab (128 bytes of K per row), so a slab's fragments are all 128
  // registers there are for them and nothing can be held twice.  A slab runs as two halves by rows of blocks -
  // half h multiplies rows [FM / 2 h, FM / 2 (h + 1)) with every column, column by column - and every fragment is
  // read again for the next slab as soon as its last MFMA of this one has been issued (an MFMA has taken its operands
  // by the time the next instruction issues, long before LDS data can come back):
  //   half 0 : the A fragments of the upper rows of THIS slab (unused in this half), and at its start the last
  //            column of B of this slab, which half 1 of the slab before was still multiplying
  //   barrier: as above
  //   half 1 : the A fragments of the lower rows of the NEXT slab, and column J - 1 of its B after the first MFMA
  //            of column J
  // so every LDS read of a slab falls between the barrier of the slab before and its own.  Half 0 starts when all
  // but the newest column asked for have come in and waits for that one and its own last column before it uses them.
  // e4m3 8192^3, us, the four-buffer kernel with the 32x32x64 instruction / this one: row/row 423 / 388, row/col
  // 438 / 376; 4096^3 on eight waves 59.9 / 52.0 and 56.4 / 51.5; 8000^2 x 8192 458 / 419 and 436 / 394.
  constexpr int HM = FM / 2 * FN;    // MFMAs per half
  auto read_a_f8 = [&](auto i_c, auto ks_c, auto jr_c) {
    constexpr int I = decltype(i_c)::value, KS = decltype(ks_c)::value, JR = decltype(jr_c)::value;
    asm_ds_read16<I * 1024>(af[KS][I], a_addr[JR][KS]);
  };
  auto read_b_col_f8 = [&](auto j_c, auto jr_c) {
    constexpr int J = decltype(j_c)::value, JR = decltype(jr_c)::value;
    if constexpr (B_KC) {
      asm_ds_read16<J * 1024>(bf[0][J], b_addr[JR][0]);
      asm_ds_read16<J * 1024>(bf[1][J], b_addr[JR][1]);
    } else {
      asm_ds_read_tr_x<ES, 0, J * TR_BLOCK_XOR>(bh[0][J][0], b_addr[(2 * JR) % NST][0]);
      asm_ds_read_tr_x<ES, TR_R_OFF, J * TR_BLOCK_XOR>(bh[0][J][1], b_addr[(2 * JR) % NST][0]);
      asm_ds_read_tr_x<ES, 0, J * TR_BLOCK_XOR>(bh[1][J][0], b_addr[(2 * JR + 1) % NST][0]);
      asm_ds_read_tr_x<ES, TR_R_OFF, J * TR_BLOCK_XOR>(bh[1][J][1], b_addr[(2 * JR + 1) % NST][0]);
    }
  };
  // after a wait: the values the MFMAs take from here on are the ones that wait was for
  auto settle_b_col_f8 = [&](auto j_c) {
    constexpr int J = decltype(j_c)::value;
    if constexpr (B_KC) asm_touch_v4(bf[0][J], bf[1][J]);
    else asm_touch_v2(bh[0][J][0], bh[0][J][1], bh[1][J][0], bh[1][J][1]);
  };
  auto mfma_f8 = [&](auto i_c, auto j_c) {
    constexpr int I = decltype(i_c)::value, J = decltype(j_c)::value;
    if constexpr (B_KC)
      asm_mfma16_f8<TYPES>(acc[I][J], join8(bf[0][J], bf[1][J]), join8(af[0][I], af[1][I]));
    else if constexpr (SWAP)
      asm_mfma16_f8<TYPES>(acc[I][J], join8(af[0][I], af[1][I]),
                           join8(join4(bh[0][J][0], bh[0][J][1]), join4(bh[1][J][0], bh[1][J][1])));
    else
      asm_mfma16_f8<TYPES>(acc[I][J], join8(join4(bh[0][J][0], bh[0][J][1]), join4(bh[1][J][0], bh[1][J][1])),
                           join8(af[0][I], af[1][I]));
  };
  // half H of the slab at ring position JR; the copies of a group of parity H into buffer CST as in kstep
  auto half_f8 = [&](auto h_c, auto jr_c, auto cst_c, const char* a_src, const char* b_src) {
    constexpr int H = decltype(h_c)::value, JR = decltype(jr_c)::value, CST = decltype(cst_c)::value;
    using NEXT = std::integral_constant<int, (JR + 1) % NST>;
    constexpr int CPE = HM / NCP;          // MFMAs per copy
    static_assert(CPE >= 2 && NCP * CPE == HM && FM == 8 && HM >= 16 && FN >= 3, "a half's copies and reads are spread over its MFMAs");
    if constexpr (H == 0) {
      // all but the reads of column FN - 2, the last that half 1 asked for (LDS reads return in order)
      if constexpr (B_KC) asm volatile("s_waitcnt lgkmcnt(2)");
      else asm volatile("s_waitcnt lgkmcnt(4)");
      static_for<FM / 2>([&](auto i_c) { asm_touch_v4(af[0][decltype(i_c)::value], af[1][decltype(i_c)::value]); });
      static_for<FN - 2>([&](auto j_c) { settle_b_col_f8(j_c); });
    } else {
      static_for<FM / 2>([&](auto i_c) { asm_touch_v4(af[0][FM / 2 + decltype(i_c)::value], af[1][FM / 2 + decltype(i_c)::value]); });
    }
    static_for<HM>([&](auto q_c) {
      constexpr int Q = decltype(q_c)::value;
      constexpr int J = Q / (FM / 2), I = H * (FM / 2) + Q % (FM / 2);
      if constexpr (H == 0 && Q == (FN - 2) * (FM / 2)) {   // the last two columns, and this half's own reads so far
        asm volatile("s_waitcnt lgkmcnt(0)");
        settle_b_col_f8(std::integral_constant<int, FN - 2>{});
        settle_b_col_f8(std::integral_constant<int, FN - 1>{});
      }
      mfma_f8(std::integral_constant<int, I>{}, std::integral_constant<int, J>{});
      if constexpr (H == 0) {
        if constexpr (Q == 0) read_b_col_f8(std::integral_constant<int, FN - 1>{}, jr_c);
        if constexpr (Q % 2 == 1 && Q / 2 < FM)   // upper rows of this slab: row FM / 2 + r / 2, K step r % 2
          read_a_f8(std::integral_constant<int, FM / 2 + (Q / 2) / 2>{}, std::integral_constant<int, (Q / 2) % 2>{}, jr_c);
      } else {
        if constexpr (Q % (FM / 2) == 0 && J >= 1) read_b_col_f8(std::integral_constant<int, J - 1>{}, NEXT{});
        if constexpr (Q % 2 == 1 && Q / 2 < FM)   // lower rows of the next slab: row r / 2, K step r % 2
          read_a_f8(std::integral_constant<int, (Q / 2) / 2>{}, std::integral_constant<int, (Q / 2) % 2>{}, NEXT{});
      }
      constexpr int Tc = Q / CPE;
      if constexpr (Q == 0) copy_a_begin(CST);
      if constexpr (Q == CPE * A_PW) copy_b_begin(CST);
      if constexpr (Q % CPE == CPE / 2) {
        if constexpr (Tc < A_PW) copy_a(std::integral_constant<int, Tc>{}, h_c, a_src);
        else copy_b(std::integral_constant<int, Tc - A_PW>{}, h_c, b_src);
      }
    });
  };

  using I0 = std::integral_constant<int, 0>;
  using I1 = std::integral_constant<int, 1>;
  // ---- prologue: groups 0 .. 3 (slabs 0 and 1; a run of one slab has groups 0 and 1 only) ----
  const char* const a_tile = a_base_of(m0);
  const char* const b_tile = b_base_of(n0);
  auto issue_group = [&](auto c_c, const char* a_t, const char* b_t) {
    constexpr int C = decltype(c_c)::value;
    const char* const a_src = a_group(a_t, C);
    const char* const b_src = b_group(b_t, C);
    copy_a_begin(C);
    static_for<A_PW>([&](auto t) { copy_a(t, std::integral_constant<int, C & 1>{}, a_src); });
    copy_b_begin(C);
    static_for<B_PW>([&](auto t) { copy_b(t, std::integral_constant<int, C & 1>{}, b_src); });
  };
  if (!(PERSISTENT && prefetched)) {   // (persistent: groups 0 and 1 went out before the last tile's epilogue)
    issue_group(std::integral_constant<int, 0>{}, a_tile, b_tile);
    issue_group(std::integral_constant<int, 1>{}, a_tile, b_tile);
  }
  // Slab 0 (groups 0 and 1) has landed; what was issued after it may still be on its way.  (Persistent: the last
  // epilogue's stores are counted between the two pairs of groups.  Loads return in order, so with no more than two
  // groups' worth of operations outstanding none of them can be a load of groups 0 and 1.)
  if (nc > 2) {
    issue_group(std::integral_constant<int, 2>{}, a_tile, b_tile);
    issue_group(std::integral_constant<int, 3>{}, a_tile, b_tile);
    asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" : : "i"(2 * NCP) : "memory");
  } else {
    asm volatile("s_waitcnt vmcnt(0)\n\ts_barrier" ::: "memory");
  }
  if constexpr (F8) {   // lower rows of A and all but the last column of B of slab 0
    static_for<FM>([&](auto r_c) {
      constexpr int R = decltype(r_c)::value;
      read_a_f8(std::integral_constant<int, R / 2>{}, std::integral_constant<int, R % 2>{}, I0{});
    });
    static_for<FN - 1>([&](auto j_c) { read_b_col_f8(j_c, I0{}); });
  } else {
    static_for<NRD>([&](auto r) { read_one(I0{}, r, I0{}); });
  }

  // ---- one slab; JR = j % 5 at compile time.  Slab j fetches slab j + 2 (groups 2j + 4 and 2j + 5) from a_cp / b_cp,
  // or, where the run has no such slab, its last slab again ----
  const int nslab = nc / 2;
  const int first_fetch = min(2, nslab - 1);
  const char* a_cp = a_group(a_tile, 2 * first_fetch);
  const char* b_cp = b_group(b_tile, 2 * first_fetch);
  auto slab = [&](auto jr_c, int j) {
    constexpr int JR = decltype(jr_c)::value;
    using NEXT = std::integral_constant<int, (JR + 1) % NST>;
    using ST4 = std::integral_constant<int, (2 * JR + 4) % NST>;
    using ST5 = std::integral_constant<int, (2 * JR + 5) % NST>;
    // a row-major B: a group is a K step's rows, the slab's second group lies a step further
    const char* const b_cp1 = B_KC ? b_cp : b_cp + b_group_step;
    const char* const a_cp1 = A_KC ? a_cp : a_cp + a_group_step;
    if constexpr (F8) half_f8(I0{}, jr_c, ST4{}, a_cp, b_cp);
    else kstep(I0{}, jr_c, I0{}, ST4{}, a_cp, b_cp);
    if (j + 2 < nslab) {  // the copies of group 2j+4 may stay in flight
      if constexpr (NCP == 8) asm volatile("s_waitcnt vmcnt(8) lgkmcnt(0)\n\ts_barrier" ::: "memory");
      else asm volatile("s_waitcnt vmcnt(4) lgkmcnt(0)\n\ts_barrier" ::: "memory");
    } else {
      asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");
    }
    if constexpr (F8) half_f8(I1{}, jr_c, ST5{}, a_cp1, b_cp1);
    else kstep(I1{}, NEXT{}, I1{}, ST5{}, a_cp1, b_cp1);
    const bool more = j + 3 < nslab;   // the next slab fetches one further
    a_cp += more ? (A_KC ? (size_t)LINE : 2 * a_group_step) : (size_t)0;
    b_cp += more ? (B_KC ? (size_t)LINE : 2 * b_group_step) : (size_t)0;
  };

  for (int j = 0; j < nslab; j += NST) {
    slab(std::integral_constant<int, 0>{}, j);
    if (j + 1 < nslab) slab(std::integral_constant<int, 1>{}, j + 1);
    if (j + 2 < nslab) slab(std::integral_constant<int, 2>{}, j + 2);
    if (j + 3 < nslab) slab(std::integral_constant<int, 3>{}, j + 3);
    if (j + 4 < nslab) slab(std::integral_constant<int, 4>{}, j + 4);
  }

  // no copy may still be in flight when the work-group ends, and the last MFMAs must have written their
  // accumulators before ordinary code reads them
  asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_nop 15\n\ts_nop 15\n\ts_nop 7" ::: "memory");
  static_for<NMMA>([&](auto q_c) {
    constexpr int Q = decltype(q_c)::value;
    asm_touch_acc4<TYPES>(acc[Q / FN][Q % FN]);
  });

  // the epilogue passes the accumulators through the end of the operand buffers: 4 and 3 and a little of 2
  constexpr int EP_COLS32 = (SWAP ? WM : WN) / 32;   // 32-column blocks of the real D per wave
  static_assert(NW * epilogue_region_bytes<EP_COLS32>() <= 3 * STAGE_BYTES, "the epilogue leaves buffers 0 and 1 alone");
  char* const staging = lds + NST * STAGE_BYTES - (NW - wave) * epilogue_region_bytes<EP_COLS32>();
  __syncthreads();   // no wave reads operands any more and no copy is in flight
  if constexpr (PERSISTENT) {
    prefetched = false;
    const int next_bid = bid + (int)gridDim.x;
    if (next_bid < tiles_m * tiles_n) {
      int tm2, tn2;
      tile_of_block(next_bid, tiles_m, tiles_n, tm2, tn2);
      const char* const a_next = a_base_of(tm2 * BM);
      const char* const b_next = b_base_of(tn2 * BN);
      if constexpr (RAGGED) set_copy_offsets(tm2 * BM, tn2 * BN);   // this tile asks for nothing more
      // into buffers 0 and 1, which the epilogue does not use
      issue_group(std::integral_constant<int, 0>{}, a_next, b_next);
      issue_group(std::integral_constant<int, 1>{}, a_next, b_next);
      prefetched = true;
    }
  }
  if constexpr (STREAMK) {
    if (partial) {
      // the sums as they are (alpha = 1, beta = 0 in the accumulator type: exact) into this piece's slot, a whole
      // 256 x 256 tile whatever M and N: rows and columns past the end hold sums of clamped rows and are not read
      constexpr int WS_TYPES = TYPES == GZ_S8S8S32 ? GZ_S8S8S32 : GZ_BF16BF16F32;
      GemmArgs<WS_TYPES> gw;
      gw.A = nullptr; gw.B = nullptr; gw.C = nullptr;
      gw.D = reinterpret_cast<typename Traits<WS_TYPES>::out_t*>(sk.ws) + (size_t)slot * STREAMK_SLOT_ELEMS;
      gw.M = BM; gw.N = BN; gw.K = K;
      gw.layoutA = g.layoutA; gw.layoutB = g.layoutB;
      gw.alpha = 1; gw.beta = 0;
      gw.store_hint = 0;
      gw.lda = K; gw.ldb = BN; gw.ldc = BN; gw.ldd = BN;
      store_accumulators_lds<WS_TYPES, WM / 32, WN / 32, false, 16>(gw, acc, wm * WM, wn * WN, lane,
                                                                    staging);
    } else {
      store_accumulators_lds<TYPES, WM / 32, WN / 32, RAGGED, 16>(g, acc, m0 + wm * WM, n0 + wn * WN, lane,
                                                                  staging);
    }
    it += nslab_seg;
    if (!partial || it >= it_end) break;
    __syncthreads();   // the next piece's copies overwrite the buffers the epilogue has just read
  } else {
    if constexpr (SWAP) {
      GemmArgs<TYPES> gr = g;   // the real output: this kernel's columns are its rows
      gr.M = g.N;
      gr.N = g.M;
      store_accumulators_lds<TYPES, WN / 32, WM / 32, RAGGED, 16, true>(gr, acc, n0 + wn * WN, m0 + wm * WM, lane, staging);
    } else {
      store_accumulators_lds<TYPES, WM / 32, WN / 32, RAGGED, 16, false, B4>(g, acc, m0 + wm * WM, n0 + wn * WN, lane,
                                                                            staging);
    }
    if constexpr (!PERSISTENT) break;
    bid += (int)gridDim.x;
    if (bid >= tiles_m * tiles_n) break;
    __syncthreads();   // the next tile's groups 2 and 3 go where the epilogue has just read
  }
  }  // pieces or tiles of this work-group
}

// Stream-K, second launch: one work-group per four rows of a stream-K tile, a lane per four columns.  The pieces of a
// tile are the runs of consecutive blocks that cover its slabs; they are added in block order.
template <int TYPES>
__global__ void __launch_bounds__(256) streamk_fixup_kernel(GemmArgs<TYPES> g, int tiles_m, int tiles_n, StreamK sk) {
  using T = Traits<TYPES>;
  using acc_t = typename T::acc_t;
  using out_t = typename T::out_t;
  const int nslab_all = g.K / (128 / (int)sizeof(typename T::in_t));
  const int tt = blockIdx.x / 64, rg = blockIdx.x % 64;
  int tm, tn;
  tile_of_lid(sk.dp_tiles + tt, tiles_m, tiles_n, tm, tn);
  const int b_first = streamk_block_of_slab(sk, tt * nslab_all), b_last = streamk_block_of_slab(sk, (tt + 1) * nslab_all - 1);
  const int r = rg * 4 + (int)threadIdx.x / 64, c = ((int)threadIdx.x % 64) * 4;
  const acc_t* ws = reinterpret_cast<const acc_t*>(sk.ws);
  acc_t sum[4] = {0, 0, 0, 0};
  for (int b = b_first; b <= b_last; b++) {
    acc_t v[4];
    __builtin_memcpy(v, ws + (size_t)(b + tt) * STREAMK_SLOT_ELEMS + (size_t)r * 256 + c, sizeof(v));
#pragma unroll
    for (int e = 0; e < 4; e++) sum[e] = b == b_first ? v[e] : sum[e] + v[e];
  }
  const int m = tm * 256 + r, n = tn * 256 + c;
  if (m >= g.M || n >= g.N) return;
  const size_t o = (size_t)m * g.ldd + n, oc = (size_t)m * g.ldc + n;
  const bool use_c = g.beta != 0;
  constexpr uintptr_t VEC_ALIGN = 4 * sizeof(out_t) - 1;
  const bool vec = n + 4 <= g.N && (g.ldd & 3) == 0 && (!use_c || (g.ldc & 3) == 0) &&
                   ((reinterpret_cast<uintptr_t>(g.D) | (use_c ? reinterpret_cast<uintptr_t>(g.C) : 0)) & VEC_ALIGN) == 0;
  if (vec) {
    out_t cv[4] = {0, 0, 0, 0}, dv[4];
    if (use_c) __builtin_memcpy(cv, g.C + oc, sizeof(cv));
#pragma unroll
    for (int e = 0; e < 4; e++) dv[e] = epilogue<TYPES>(sum[e], g.alpha, g.beta, &cv[e]);
    __builtin_memcpy(g.D + o, dv, sizeof(dv));
  } else {
#pragma unroll
    for (int e = 0; e < 4; e++)
      if (n + e < g.N) g.D[o + e] = epilogue<TYPES>(sum[e], g.alpha, g.beta, g.C + oc + e);
  }
}

}  // namespace gz
