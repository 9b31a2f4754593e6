// MFMA rung, deep-pipeline fast path: four LDS buffers of 64-byte K rows.
//
// Why four buffers.  Moving a K slab from L2 into LDS takes the texture path most of the time the matrix
// pipe needs to consume it, and a direct-to-LDS copy lands 1000-1500 cycles after it is issued.  With two
// 128-byte buffers a copy can only start when its buffer has been drained and must have landed one slab
// later, so either the copies are bunched right after the barrier (and the waves, which issue in order,
// stall behind them) or the last ones are waited for.  Halving the K extent of a buffer (64 bytes per
// row: 32 16-bit elements or 64 int8, two MFMA steps) and keeping four of them lets every copy be issued
// evenly - four per wave and MFMA step - a full three half-slabs before its data is needed.
//
// Per half-slab h (buffer h % 4):
//   step 0 : MFMAs on the fragments of (h, step 0); requests the fragments of (h, step 1);
//            issues the B-row copies of half-slab h+3 into buffer (h+3) % 4
//   barrier: lgkmcnt(0) - this wave has finished reading buffer h % 4, which is free afterwards;
//            vmcnt(2n)  - this wave's copies of half-slab h+1 have landed (the 2n issued later may fly,
//                         n = copies per wave and half-slab)
//   step 1 : MFMAs on (h, step 1); requests the fragments of (h+1, step 0) from buffer (h+1) % 4;
//            issues the A-row copies of half-slab h+4 into buffer h % 4
// One memory instruction follows each MFMA; the sequence is fixed with asm statements (see mfma_asm_kernel).
//
// LDS rows are unpadded 64-byte rows; chunk c (16 bytes) of tile row r lives at position c ^ ((r >> 2) & 3),
// which spreads 16 consecutive rows over the 16 four-bank groups of a 64-bank line.
//
// B_KC = false: B is row-major (N contiguous), the layout of the reference's own drivers.  Its half-slab then
// sits in LDS as K rows of BN elements, filled by the same 1 KiB copies (whole K rows, so the global reads are
// long contiguous runs), and the MFMA fragments - which want 8 (16 for int8) consecutive K values of one column
// per lane - come out of LDS through the transposing reads ds_read_b64_tr_b16 / ds_read_b64_tr_b8: within 16
// lanes, lane i supplies the address of 8 bytes of a [4 x 16] (b16) or [8 x 16] (b8) block, row by row, and
// receives column i.  Two such reads make one fragment.  16-byte pieces of K row r are stored at position
// piece ^ f(r), f(r) = (r & 3) << 2 (b16) or (r & 7) << 1 (b8), so that the rows a read touches fall into
// different banks.
#pragma once

namespace gz {

__device__ inline int pipe4_swz(int r) { return (r >> 2) & 3; }

template <int ES, int OFF> __device__ __forceinline__ void asm_ds_read_tr(u32x2_t& dst, uint32_t addr) {
  if constexpr (ES == 2) asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "i"(OFF));
  else asm volatile("ds_read_b64_tr_b8 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "i"(OFF));
}

// copy with a lane mask: an all-zero mask turns the instruction into a no-op that still takes its place in
// the sequence (and in the vmcnt order)
template <int OFF>
__device__ __forceinline__ void asm_copy16_masked(uint32_t voff, const void* sbase_minus_off, uint64_t mask) {
  static_assert(OFF >= -4096 && OFF <= 4095, "13-bit signed immediate");
  asm volatile("s_mov_b64 exec, %3\n\tglobal_load_lds_dwordx4 %0, %1 offset:%2\n\ts_mov_b64 exec, -1"
               :
               : "v"(voff), "s"(sbase_minus_off), "i"(OFF), "s"(mask)
               : "memory");
}

template <int TYPES, int BM, int BN, int WAVES_M, int WAVES_N, bool B_KC = true, bool RAGGED = false>
__global__ void __launch_bounds__(WAVES_M* WAVES_N * 64)
    mfma_pipe4_kernel(GemmArgs<TYPES> g, int tiles_m, int tiles_n) {
  using T = Traits<TYPES>;
  using in_t = typename T::in_t;
  using out_t = typename T::out_t;
  using acc_v = typename AccVec<TYPES>::type;
  constexpr int NW = WAVES_M * WAVES_N;
  constexpr int ES = (int)sizeof(in_t);
  constexpr int EPV = 16 / ES;
  constexpr int ROWB = 64;            // K bytes per row and buffer
  constexpr int HK = ROWB / ES;       // K elements per half-slab
  constexpr int NST = 4;              // LDS buffers
  constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;
  constexpr int FM = WM / 32, FN = WN / 32;
  constexpr int NMMA = FM * FN, NRD = B_KC ? FM + FN : FM + 2 * FN;  // LDS reads per MFMA step
  constexpr int A_BYTES = BM * ROWB, B_BYTES = BN * ROWB;
  constexpr int STAGE_BYTES = A_BYTES + B_BYTES;
  constexpr int A_PW = BM / 16 / NW, B_PW = BN / 16 / NW;  // 1 KiB copies (16 rows) per wave and half-slab
  constexpr int NCP = A_PW + B_PW;
  static_assert(BM % (16 * NW) == 0 && BN % (16 * NW) == 0, "tile rows must divide over the waves");
  static_assert(A_PW <= 8 && B_PW <= 8 && A_PW % 2 == 0 && B_PW % 2 == 0, "a copy group must fit the immediate offset range");
  static_assert(NCP == 8 || NCP == 4, "the vmcnt immediates below are written out for 8 or 4 copies per wave and half-slab");

  extern __shared__ __attribute__((aligned(1024))) char lds[];
  const uint32_t lds_base = (uint32_t)(uintptr_t)lds;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave % WAVES_M, wn = wave / WAVES_M;
  int tm, tn;
  tile_of_block(blockIdx.x, tiles_m, tiles_n, tm, tn);
  const int m0 = tm * BM, n0 = tn * BN;
  const int K = g.K;
  const int nh = K / HK;  // half-slabs, >= 2 on this path

  // ---- copy addressing: lane -> (row lr of a 16-row group, LDS position lp) ----
  const int lr = lane >> 2, lp = lane & 3;
  const uint32_t voff = (uint32_t)((lr * K + (lp ^ pipe4_swz(lr)) * EPV) * ES);
  const char* a_ubase = reinterpret_cast<const char*>(g.A) + (size_t)(m0 + 16 * wave * A_PW) * K * ES;
  const size_t group_step = (size_t)16 * K * ES;
  // row-major B: a copy moves KRC whole K rows of the tile (BN elements each); lane -> (row, 16-byte position)
  constexpr int KRC = 1024 / (BN * ES), LPR = 64 / KRC;  // K rows per copy, lanes per row
  const int N = g.N;
  uint32_t voff_b[2] = {0, 0};
  const char* b_ubase;
  size_t b_copy_step, b_half_step;
  if constexpr (B_KC) {
    b_ubase = reinterpret_cast<const char*>(g.B) + (size_t)(n0 + 16 * wave * B_PW) * K * ES;
    b_copy_step = group_step;
    b_half_step = ROWB;
  } else {
    static_assert(B_KC || (KRC * BN * ES == 1024 && B_PW % 2 == 0), "whole K rows per copy");
#pragma unroll
    for (int par = 0; par < 2; par++) {  // copy t of the wave: rows KRC (wave B_PW + t) .., parity of t decides f(row)
      const int kr = KRC * par + lane / LPR;   // row within a pair of copies; wave * B_PW * KRC is a multiple of 8
      const int f = ES == 2 ? (kr & 3) << 2 : (kr & 7) << 1;
      voff_b[par] = (uint32_t)(((size_t)(lane / LPR) * N + (size_t)(((lane % LPR) ^ f) * EPV)) * ES);
    }
    b_ubase = reinterpret_cast<const char*>(g.B) + ((size_t)(wave * B_PW * KRC) * N + n0) * ES;
    b_copy_step = (size_t)KRC * N * ES;
    b_half_step = (size_t)HK * N * ES;
  }
  // RAGGED: M and N need not be multiples of the tile (K still a whole number of slabs, rows 16-byte aligned).  Rows
  // past the end are fetched from the last row (columns of a row-major B from its last 16-byte piece): an output
  // depends on its own row of A and column of B only, and those past the end are not stored.  The per-copy offsets
  // are then relative to the tile's first row instead of the copy's.
  const int M = g.M;
  uint32_t voff_ar[RAGGED ? A_PW : 1], voff_br[RAGGED && B_KC ? B_PW : 1];
  const char* a_tile = reinterpret_cast<const char*>(g.A) + (size_t)m0 * K * ES;
  const char* b_tile = reinterpret_cast<const char*>(g.B) + (size_t)n0 * K * ES;
  if constexpr (RAGGED) {
#pragma unroll
    for (int t = 0; t < A_PW; t++) {
      const int rc = min(m0 + 16 * (wave * A_PW + t) + lr, M - 1) - m0;
      voff_ar[t] = (uint32_t)(((size_t)rc * K + (size_t)((lp ^ pipe4_swz(lr)) * EPV)) * ES);
    }
    if constexpr (B_KC) {
#pragma unroll
      for (int t = 0; t < B_PW; t++) {
        const int rc = min(n0 + 16 * (wave * B_PW + t) + lr, N - 1) - n0;
        voff_br[t] = (uint32_t)(((size_t)rc * K + (size_t)((lp ^ pipe4_swz(lr)) * EPV)) * ES);
      }
    } else {
      const int last_piece = (N - n0) / EPV - 1;   // N is a multiple of EPV on this path, n0 < N
#pragma unroll
      for (int par = 0; par < 2; par++) {
        const int kr = KRC * par + lane / LPR;
        const int f = ES == 2 ? (kr & 3) << 2 : (kr & 7) << 1;
        voff_b[par] = (uint32_t)(((size_t)(lane / LPR) * N + (size_t)(min((lane % LPR) ^ f, last_piece) * EPV)) * ES);
      }
    }
  }
  // A-row copies of half-slab hs into buffer st (one M0 for the group)
  auto copy_a_begin = [&](int st) { asm_set_m0(lds_base + st * STAGE_BYTES + (wave * A_PW) * 1024 + (A_PW / 2) * 1024); };
  auto copy_b_begin = [&](int st) {
    asm_set_m0(lds_base + st * STAGE_BYTES + A_BYTES + (wave * B_PW) * 1024 + (B_PW / 2) * 1024);
  };
  auto copy_a = [&](auto t_c, int hs, uint64_t mask) {
    constexpr int Tn = decltype(t_c)::value, OFF = (Tn - A_PW / 2) * 1024;
    if constexpr (RAGGED) asm_copy16_masked<OFF>(voff_ar[Tn], a_tile + (size_t)hs * ROWB - OFF, mask);
    else asm_copy16_masked<OFF>(voff, a_ubase + Tn * group_step + (size_t)hs * ROWB - OFF, mask);
  };
  auto copy_b = [&](auto t_c, int hs, uint64_t mask) {
    constexpr int Tn = decltype(t_c)::value, OFF = (Tn - B_PW / 2) * 1024;
    if constexpr (RAGGED && B_KC) asm_copy16_masked<OFF>(voff_br[Tn], b_tile + (size_t)hs * ROWB - OFF, mask);
    else asm_copy16_masked<OFF>(B_KC ? voff : voff_b[Tn & 1], b_ubase + Tn * b_copy_step + (size_t)hs * b_half_step - OFF, mask);
  };

  // ---- fragment addressing: one LDS byte address per (buffer, step) ----
  const int frag_row = lane & 31, half = lane >> 5;
  const int sw = pipe4_swz(frag_row);
  uint32_t a_addr[NST][2], b_addr[NST][B_KC ? 2 : FN];
#pragma unroll
  for (int st = 0; st < NST; st++)
#pragma unroll
    for (int ks = 0; ks < 2; ks++) {
      const int pos = ((ks * 2 + half) ^ sw) * 16;
      a_addr[st][ks] = lds_base + st * STAGE_BYTES + (wm * WM + frag_row) * ROWB + pos;
      if constexpr (B_KC) b_addr[st][ks] = lds_base + st * STAGE_BYTES + A_BYTES + (wn * WN + frag_row) * ROWB + pos;
    }
  // transposing reads: lane i of a 16-lane group addresses row fi of the block's K rows and the piece of 8 bytes
  // that holds columns 16 (group & 1) + (4 or 8) (i % lanes-per-row); groups 2, 3 take the upper half of the K step.
  // One address per (buffer, 32-column block); K step and half fragment go into the immediate offset.
  constexpr int TR_LPR = ES == 2 ? 4 : 2;            // lanes per K row within a 16-lane group
  constexpr int TR_PITCH = BN * ES;                   // bytes per K row
  constexpr int TR_KS_OFF = (16 / ES * 2) * TR_PITCH; // next MFMA step: 16 (32) K rows further
  constexpr int TR_R_OFF = (16 / TR_LPR) * TR_PITCH;  // second half fragment: 4 (8) K rows further
  if constexpr (!B_KC) {
    static_assert(B_KC || (TR_KS_OFF + TR_R_OFF < 65536 && TR_KS_OFF == B_BYTES / 2), "immediate offsets");
    const int i16 = lane & 15, fi = i16 / TR_LPR;
    const int n_sub = ((lane >> 4) & 1) * 16 + (i16 % TR_LPR) * (8 / ES);   // column within the 32-column block
    const int krow = (lane >> 5) * (16 / TR_LPR * 2) + fi;                  // K row within the MFMA step
    const int f = ES == 2 ? (fi & 3) << 2 : (fi & 7) << 1;
#pragma unroll
    for (int st = 0; st < NST; st++)
#pragma unroll
      for (int j = 0; j < FN; j++) {
        const int n_local = wn * WN + j * 32 + n_sub;
        const int piece = (n_local / EPV) ^ f;
        b_addr[st][j] = lds_base + st * STAGE_BYTES + A_BYTES + krow * TR_PITCH + piece * 16 + (n_local % EPV) * ES;
      }
  }

  acc_v acc[FM][FN];
#pragma unroll
  for (int i = 0; i < FM; i++)
#pragma unroll
    for (int j = 0; j < FN; j++)
#pragma unroll
      for (int v = 0; v < 16; v++) acc[i][j][v] = 0;
  static_for<NMMA>([&](auto q_c) {
    constexpr int Q = decltype(q_c)::value;
    asm_touch_acc<TYPES>(acc[Q / FN][Q % FN]);
  });
  asm volatile("s_nop 7" ::: "memory");
  // Register sets of fragments: one per MFMA step.  The 8-bit float types use v_mfma_f32_32x32x64_f8f6f4, whose
  // operands are the fragments of both steps of a half-slab side by side, so they keep four sets: set 2 P + ks holds
  // step ks of the half-slabs of parity P.
  constexpr bool F8 = is_fp8(TYPES);
  // (The same half-slab-ahead schedule works for the other types, one step's MFMAs per part; measured against
  // hipBLASLt in the same run it changed bf16 4096^3 by -1 % and int8 8192^3 by +2 %, so they keep two sets.)
  constexpr bool DEEP = F8;
  constexpr int NSETS = DEEP ? 4 : 2;
  u32x4_t af[NSETS][FM], bf[NSETS][FN];
  u32x2_t bh[NSETS][FN][2];  // row-major B: the two halves of a fragment as they come out of the transposing reads

  auto read_one = [&](auto set_c, auto r_c, int st, int ks) {
    constexpr int SET = decltype(set_c)::value, R = decltype(r_c)::value;
    if constexpr (R < FM) {
      asm_ds_read16<R * 32 * ROWB>(af[SET][R], a_addr[st][ks]);
    } else if constexpr (B_KC) {
      asm_ds_read16<(R - FM) * 32 * ROWB>(bf[SET][R - FM], b_addr[st][ks]);
    } else {
      constexpr int J = (R - FM) / 2, HALF = (R - FM) % 2;
      if (ks == 0) asm_ds_read_tr<ES, HALF * TR_R_OFF>(bh[SET][J][HALF], b_addr[st][J]);
      else asm_ds_read_tr<ES, TR_KS_OFF + HALF * TR_R_OFF>(bh[SET][J][HALF], b_addr[st][J]);
    }
  };

  // One MFMA step: NMMA MFMAs on register set SET; after MFMA q the q-th memory instruction of the step:
  // first the NRD fragment reads of (buffer rst, step rks) into the other set, then this step's copies.
  auto step = [&](auto set_c, int rst, int rks, auto copy_is_a, int cst, int chs, uint64_t cmask) {
    constexpr int SET = decltype(set_c)::value;
    constexpr bool IS_A = decltype(copy_is_a)::value;
    constexpr int NC = IS_A ? A_PW : B_PW;
    constexpr int NOPS = NRD + NC;
    static_assert(NOPS <= NMMA, "one memory instruction per MFMA");
    asm volatile("s_waitcnt lgkmcnt(0)");
    if constexpr (!B_KC) {
#pragma unroll
      for (int j = 0; j < FN; j++) {
        asm volatile("" : "+v"(bh[SET][j][0]), "+v"(bh[SET][j][1]));  // after the wait
        bf[SET][j] = u32x4_t{bh[SET][j][0][0], bh[SET][j][0][1], bh[SET][j][1][0], bh[SET][j][1][1]};
      }
    }
    if constexpr (IS_A) copy_a_begin(cst);
    else copy_b_begin(cst);
    static_for<NMMA>([&](auto q_c) {
      constexpr int Q = decltype(q_c)::value;
      asm_mfma32<TYPES>(acc[Q / FN][Q % FN], bf[SET][Q % FN], af[SET][Q / FN]);
      if constexpr (Q < NRD) {
        read_one(std::integral_constant<int, SET ^ 1>{}, q_c, rst, rks);
      } else if constexpr (Q < NOPS) {
        if constexpr (IS_A) copy_a(std::integral_constant<int, Q - NRD>{}, chs, cmask);
        else copy_b(std::integral_constant<int, Q - NRD>{}, chs, cmask);
      }
    });
  };

  // 8-bit floats: half a half-slab's MFMAs (each covers both K steps: 64 K values, 16 passes) on the sets of parity P;
  // meanwhile the fragments of (buffer rst, step PART) go to the sets of the other parity and this part's copies are
  // issued, up to two memory instructions after each MFMA.  The fragments were waited for at the barrier.
  auto step_f8 = [&](auto p_c, auto part_c, int rst, auto copy_is_a, int cst, int chs, uint64_t cmask) {
    constexpr int P = decltype(p_c)::value, PART = decltype(part_c)::value;
    constexpr bool IS_A = decltype(copy_is_a)::value;
    constexpr int NC = IS_A ? A_PW : B_PW;
    constexpr int NOPS = NRD + NC, PART_MMA = F8 ? NMMA / 2 : NMMA;
    constexpr int PER = (NOPS + PART_MMA - 1) / PART_MMA;
    static_assert(PER <= 2, "at most two memory instructions per MFMA");
    if constexpr (!B_KC && (PART == 0 || !F8)) {
#pragma unroll
      for (int ks = F8 ? 0 : PART; ks < (F8 ? 2 : PART + 1); ks++)
#pragma unroll
        for (int j = 0; j < FN; j++) {
          asm volatile("" : "+v"(bh[2 * P + ks][j][0]), "+v"(bh[2 * P + ks][j][1]));  // after the wait
          bf[2 * P + ks][j] = u32x4_t{bh[2 * P + ks][j][0][0], bh[2 * P + ks][j][0][1], bh[2 * P + ks][j][1][0],
                                      bh[2 * P + ks][j][1][1]};
        }
    }
    if constexpr (IS_A) copy_a_begin(cst);
    else copy_b_begin(cst);
    static_for<PART_MMA>([&](auto q_c) {
      constexpr int QL = decltype(q_c)::value, Q = F8 ? PART * PART_MMA + QL : QL;
      if constexpr (F8)
        asm_mfma_f8<TYPES>(acc[Q / FN][Q % FN], bf[2 * P][Q % FN], bf[2 * P + 1][Q % FN], af[2 * P][Q / FN],
                           af[2 * P + 1][Q / FN]);
      else
        asm_mfma32<TYPES>(acc[Q / FN][Q % FN], bf[2 * P + PART][Q % FN], af[2 * P + PART][Q / FN]);
      static_for<PER>([&](auto o_c) {
        constexpr int OP = QL * PER + decltype(o_c)::value;
        if constexpr (OP < NRD) {
          read_one(std::integral_constant<int, 2 * (P ^ 1) + PART>{}, std::integral_constant<int, OP>{}, rst, PART);
        } else if constexpr (OP < NOPS) {
          if constexpr (IS_A) copy_a(std::integral_constant<int, OP - NRD>{}, chs, cmask);
          else copy_b(std::integral_constant<int, OP - NRD>{}, chs, cmask);
        }
      });
    });
  };

  const std::true_type is_a{};
  const std::false_type is_b{};
  using I0 = std::integral_constant<int, 0>;
  using I1 = std::integral_constant<int, 1>;
  // lane mask of a copy as a scalar register pair: all ones while the half-slab exists, zero past the end
  auto mask_if = [](bool on) -> uint64_t {
    const uint32_t w = (uint32_t)__builtin_amdgcn_readfirstlane(on ? -1 : 0);
    return ((uint64_t)w << 32) | w;
  };

  // ---- prologue: half-slabs 0, 1, 2 whole and the A rows of 3 ----
  static_for<3>([&](auto h_c) {
    constexpr int H = decltype(h_c)::value;
    const uint64_t m = mask_if(H < nh);
    copy_a_begin(H);
    static_for<A_PW>([&](auto t) { copy_a(t, H, m); });
    copy_b_begin(H);
    static_for<B_PW>([&](auto t) { copy_b(t, H, m); });
  });
  copy_a_begin(3);
  {
    const uint64_t m3 = mask_if(3 < nh);
    static_for<A_PW>([&](auto t) { copy_a(t, 3, m3); });
    if constexpr (DEEP) {  // the 8-bit float pipeline runs half a half-slab earlier: all of half-slab 3 here
      copy_b_begin(3);
      static_for<B_PW>([&](auto t) { copy_b(t, 3, m3); });
    }
  }
  // half-slab 0 has landed (what was issued after it may still be on its way: the first barriers of the loop wait
  // for the following half-slabs in turn)
  asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" : : "i"(DEEP ? 3 * NCP : 2 * NCP + A_PW) : "memory");
  static_for<NRD>([&](auto r) { read_one(I0{}, r, 0, 0); });
  if constexpr (DEEP) static_for<NRD>([&](auto r) { read_one(I1{}, r, 0, 1); });

  // ---- one half-slab; S = h % 4 at compile time ----
  auto half_slab = [&](auto s_c, int h) {
    constexpr int S = decltype(s_c)::value;
    if constexpr (DEEP) {
      // barrier first: this wave has the fragments of half-slab h (both steps), so buffer S is free once every wave
      // is here, and its copies of half-slab h+1 have landed (the 2 * NCP issued after them may stay in flight)
      if (h + 3 < nh) {
        if constexpr (NCP == 8) asm volatile("s_waitcnt vmcnt(16) lgkmcnt(0)\n\ts_barrier" ::: "memory");
        else asm volatile("s_waitcnt vmcnt(8) lgkmcnt(0)\n\ts_barrier" ::: "memory");
      } else {
        asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");
      }
      const uint64_t m4 = mask_if(h + 4 < nh);
      step_f8(std::integral_constant<int, S & 1>{}, I0{}, (S + 1) % NST, is_b, S, h + 4, m4);
      step_f8(std::integral_constant<int, S & 1>{}, I1{}, (S + 1) % NST, is_a, S, h + 4, m4);
    } else {
      step(I0{}, S, 1, is_b, (S + 3) % NST, h + 3, mask_if(h + 3 < nh));
      if (h + 3 < nh) {  // the 2 * NCP copies issued after those of half-slab h+1 may stay in flight
        if constexpr (NCP == 8) asm volatile("s_waitcnt vmcnt(16) lgkmcnt(0)\n\ts_barrier" ::: "memory");
        else asm volatile("s_waitcnt vmcnt(8) lgkmcnt(0)\n\ts_barrier" ::: "memory");
      } else {
        asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");
      }
      step(I1{}, (S + 1) % NST, 0, is_a, S, h + 4, mask_if(h + 4 < nh));
    }
  };

  for (int h = 0; h < nh; h += 4) {
    half_slab(std::integral_constant<int, 0>{}, h);
    if (h + 1 < nh) half_slab(std::integral_constant<int, 1>{}, h + 1);
    if (h + 2 < nh) half_slab(std::integral_constant<int, 2>{}, h + 2);
    if (h + 3 < nh) half_slab(std::integral_constant<int, 3>{}, h + 3);
  }

  // no copy may still be in flight when the work-group ends, and the last MFMAs must have written their
  // accumulators before ordinary code reads them
  asm volatile("s_waitcnt vmcnt(0)\n\ts_nop 15\n\ts_nop 15\n\ts_nop 7" ::: "memory");
  static_for<NMMA>([&](auto q_c) {
    constexpr int Q = decltype(q_c)::value;
    asm_touch_acc<TYPES>(acc[Q / FN][Q % FN]);
  });

  static_assert(NW * epilogue_region_bytes<FN>() <= NST * STAGE_BYTES, "the epilogue reuses the operand buffers");
  __syncthreads();   // no wave reads operands any more and no copy is in flight
  store_accumulators_lds<TYPES, FM, FN, RAGGED>(g, acc, m0 + wm * WM, n0 + wn * WN, lane, lds + wave * epilogue_region_bytes<FN>());
}

}  // namespace gz
