// MFMA rung, whole-line variant of the deep-pipeline fast path: a ring of five LDS buffers, slabs cut by rows.
//
// mfma_pipe4_kernel cuts a K slab of 128 bytes per row into two half-slabs of 64 bytes, so each of its copies asks
// L2 for half a cache line and the other half is asked for one half-slab later: twice the requests the data needs.
// Here the eight lanes that fill one row of a copy ask for one whole 128-byte line, and a slab is cut the other way:
// copy group c carries, for slab c / 2 (all four MFMA steps of it), the rows r of every 16-row group of the tile
// with (r >> 3) & 1 == c & 1.  A slab can be multiplied only when both of its groups have landed, so the pipeline
// runs by slabs, and since a group's buffer stays busy for the whole slab a ring of five buffers (all 160 KiB) is
// what keeps one copy batch per MFMA step:
//
// Per slab j (groups 2j and 2j+1 in buffers (2j) % 5 and (2j+1) % 5), four MFMA steps:
//   step 0 : MFMAs on (j, step 0); requests the fragments of (j, 1); issues the A rows of group 2j+4
//   step 1 : MFMAs on (j, 1); requests (j, 2); issues the B rows of group 2j+4
//   step 2 : MFMAs on (j, 2); requests (j, 3)
//   barrier: lgkmcnt(0) - this wave has finished reading slab j, whose two buffers are free afterwards;
//            vmcnt(n)   - this wave's copies of groups 2j+2 and 2j+3 have landed (the n of group 2j+4 may fly,
//                         n = copies per wave and group)
//   step 3 : MFMAs on (j, 3); requests (j+1, 0); issues all of group 2j+5 into buffer (2j) % 5, which the barrier
//            has just freed: the odd group has the shortest way to the barrier that needs it (three steps), so it
//            goes out at once, up to two memory instructions after an MFMA
// Elsewhere one memory instruction follows each MFMA, as in mfma_pipe4_kernel.  (EARLY_ODD = false spreads the
// odd group over step 3 and the next step 0 instead, one instruction per MFMA throughout: 0.7-0.9 % slower with
// eight waves, bf16 4096^3 108.8 against 107.9 us, 8192^3 792 against 785; no difference with four.)
//
// LDS: a copy fills 1 KiB with 8 rows of 128 bytes; 16-byte piece c of the row with index i (0..7) within its
// copy and group parity p lives at slot c ^ i ^ p, so that the 16 rows which 16 consecutive lanes of a fragment
// read touch fall into the 16 four-bank groups of a 64-bank line.
//
// K a multiple of the slab (128 bytes), A row-major; whole tiles, or (RAGGED, column-major B) any M and N with
// 16-byte aligned rows.  B_KC = false: B is row-major; its copies move
// whole K rows already, so group c simply carries K rows [h c, h c + h) of B (h = 32 16-bit or 64 int8 rows) in
// mfma_pipe4_kernel's layout, read through the transposing LDS reads: MFMA step s of a slab finds its B rows in the
// group of parity s / 2.
#pragma once

#ifndef GZ_RING5_EARLY_ODD
#define GZ_RING5_EARLY_ODD true
#endif

namespace gz {

template <int TYPES, int BM, int BN, int WAVES_M, int WAVES_N, bool B_KC = true, bool RAGGED = false, bool EARLY_ODD = GZ_RING5_EARLY_ODD>
__global__ void __launch_bounds__(WAVES_M* WAVES_N * 64)
    mfma_ring5_kernel(GemmArgs<TYPES> g, int tiles_m, int tiles_n) {
  using T = Traits<TYPES>;
  using in_t = typename T::in_t;
  using acc_v = typename AccVec<TYPES>::type;
  constexpr int NW = WAVES_M * WAVES_N;
  constexpr int ES = (int)sizeof(in_t);
  constexpr int LINE = 128;           // K bytes per row and slab
  constexpr int SK = LINE / ES;       // K elements per slab
  constexpr int NST = 5;              // LDS buffers, one copy group each
  constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;
  constexpr int FM = WM / 32, FN = WN / 32;
  constexpr int EPV = 16 / ES;
  constexpr int HK = 64 / ES;         // K rows of a row-major B per copy group
  constexpr int NMMA = FM * FN, NRD = B_KC ? FM + FN : FM + 2 * FN;  // LDS reads per MFMA step
  constexpr int A_BYTES = BM / 2 * LINE, B_BYTES = BN / 2 * LINE;
  constexpr int STAGE_BYTES = A_BYTES + B_BYTES;
  constexpr int A_PW = BM / 16 / NW, B_PW = BN / 16 / NW;  // 1 KiB copies (8 rows) per wave and group
  constexpr int NCP = A_PW + B_PW;
  static_assert(!is_fp8(TYPES) && TYPES != GZ_F32F32F32, "16-bit and int8 operands");
  static_assert(B_KC || !RAGGED, "ragged grids with a column-major B only");
  static_assert(BM % (16 * NW) == 0 && BN % (16 * NW) == 0, "tile rows must divide over the waves");
  static_assert(A_PW <= 8 && B_PW <= 8 && A_PW % 2 == 0 && B_PW % 2 == 0, "a copy group must fit the immediate offset range");
  static_assert(NCP == 8 || NCP == 4, "the vmcnt immediates below are written out for 8 or 4 copies per wave and group");

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
  const int nc = 2 * (K / SK);  // copy groups

  // ---- copy addressing: lane -> (row ci of the 8 rows of a copy, LDS slot cs); one offset per group parity ----
  const int ci = lane >> 3, cs = lane & 7;
  const uint32_t voff[2] = {(uint32_t)(ci * K * ES + ((cs ^ ci) * 16)), (uint32_t)(ci * K * ES + ((cs ^ ci ^ 1) * 16))};
  const size_t group_step = (size_t)16 * K * ES, parity_step = (size_t)8 * K * ES;
  const char* a_ubase = reinterpret_cast<const char*>(g.A) + (size_t)(m0 + 16 * wave * A_PW) * K * ES;
  // row-major B: group c carries K rows [HK c, HK c + HK) of B, BN elements each, as mfma_pipe4_kernel lays them out:
  // a copy moves KRC whole K rows; lane -> (row, 16-byte position), pieces of K row r at position piece ^ f(r)
  constexpr int KRC = 1024 / (BN * ES), LPR = 64 / KRC;
  const int N = g.N;
  uint32_t voff_b[2] = {0, 0};
  const char* b_ubase;
  size_t b_copy_step = 0, b_group_step = 0;
  if constexpr (B_KC) {
    b_ubase = reinterpret_cast<const char*>(g.B) + (size_t)(n0 + 16 * wave * B_PW) * K * ES;
  } else {
    static_assert(B_KC || (KRC * BN * ES == 1024 && B_PW % 2 == 0), "whole K rows per copy");
#pragma unroll
    for (int par = 0; par < 2; par++) {
      const int kr = KRC * par + lane / LPR;
      const int f = ES == 2 ? (kr & 3) << 2 : (kr & 7) << 1;
      voff_b[par] = (uint32_t)(((size_t)(lane / LPR) * N + (size_t)(((lane % LPR) ^ f) * EPV)) * ES);
    }
    b_ubase = reinterpret_cast<const char*>(g.B) + ((size_t)(wave * B_PW * KRC) * N + n0) * ES;
    b_copy_step = (size_t)KRC * N * ES;
    b_group_step = (size_t)HK * N * ES;
  }
  // RAGGED: M and N need not be multiples of the tile.  Rows past the end are fetched from the last row: an output
  // depends on its own row of A and column of B only, and those past the end are not stored.  The per-copy offsets
  // are then relative to the tile's first row instead of the copy's.
  uint32_t voff_ar[2][RAGGED ? A_PW : 1], voff_br[2][RAGGED ? B_PW : 1];
  const char* a_tile = reinterpret_cast<const char*>(g.A) + (size_t)m0 * K * ES;
  const char* b_tile = reinterpret_cast<const char*>(g.B) + (size_t)n0 * K * ES;
  if constexpr (RAGGED) {
#pragma unroll
    for (int par = 0; par < 2; par++) {
#pragma unroll
      for (int t = 0; t < A_PW; t++) {
        const int rc = min(m0 + 16 * (wave * A_PW + t) + 8 * par + ci, g.M - 1) - m0;
        voff_ar[par][t] = (uint32_t)((size_t)rc * K * ES + (size_t)((cs ^ ci ^ par) * 16));
      }
#pragma unroll
      for (int t = 0; t < B_PW; t++) {
        const int rc = min(n0 + 16 * (wave * B_PW + t) + 8 * par + ci, g.N - 1) - n0;
        voff_br[par][t] = (uint32_t)((size_t)rc * K * ES + (size_t)((cs ^ ci ^ par) * 16));
      }
    }
  }
  auto copy_a_begin = [&](int st) { asm_set_m0(lds_base + st * STAGE_BYTES + (wave * A_PW) * 1024 + (A_PW / 2) * 1024); };
  auto copy_b_begin = [&](int st) {
    asm_set_m0(lds_base + st * STAGE_BYTES + A_BYTES + (wave * B_PW) * 1024 + (B_PW / 2) * 1024);
  };
  // copy t of this wave for group c (parity P = c & 1 at compile time)
  auto copy_a = [&](auto t_c, auto p_c, int c, uint64_t mask) {
    constexpr int Tn = decltype(t_c)::value, P = decltype(p_c)::value, OFF = (Tn - A_PW / 2) * 1024;
    if constexpr (RAGGED) asm_copy16_masked<OFF>(voff_ar[P][Tn], a_tile + (size_t)(c >> 1) * LINE - OFF, mask);
    else asm_copy16_masked<OFF>(voff[P], a_ubase + Tn * group_step + P * parity_step + (size_t)(c >> 1) * LINE - OFF, mask);
  };
  auto copy_b = [&](auto t_c, auto p_c, int c, uint64_t mask) {
    constexpr int Tn = decltype(t_c)::value, P = decltype(p_c)::value, OFF = (Tn - B_PW / 2) * 1024;
    if constexpr (RAGGED) asm_copy16_masked<OFF>(voff_br[P][Tn], b_tile + (size_t)(c >> 1) * LINE - OFF, mask);
    else if constexpr (B_KC) asm_copy16_masked<OFF>(voff[P], b_ubase + Tn * group_step + P * parity_step + (size_t)(c >> 1) * LINE - OFF, mask);
    else asm_copy16_masked<OFF>(voff_b[Tn & 1], b_ubase + Tn * b_copy_step + (size_t)c * b_group_step - OFF, mask);
  };

  // ---- fragment addressing: one LDS byte address per (slab position in the ring, step) ----
  // tile row r = 16 G + 8 p + i lives in the buffer of group parity p at G * 1024 + i * 128
  const int frag_row = lane & 31, half = lane >> 5;
  const int fp = (frag_row >> 3) & 1, fi = frag_row & 7;
  uint32_t a_addr[NST][4], b_addr[NST][B_KC ? 4 : FN];  // row-major B: per (buffer, 32-column block)
#pragma unroll
  for (int jr = 0; jr < NST; jr++) {
    const int buf = (2 * jr + fp) % NST;
#pragma unroll
    for (int ks = 0; ks < 4; ks++) {
      const int pos = ((ks * 2 + half) ^ fi ^ fp) * 16;
      a_addr[jr][ks] = lds_base + buf * STAGE_BYTES + (wm * WM / 16 + (frag_row >> 4)) * 1024 + fi * LINE + pos;
      if constexpr (B_KC)
        b_addr[jr][ks] = lds_base + buf * STAGE_BYTES + A_BYTES + (wn * WN / 16 + (frag_row >> 4)) * 1024 + fi * LINE + pos;
    }
  }

  // transposing reads of a row-major B (see mfma_pipe4_kernel): one address per (buffer, 32-column block); K step
  // within the group and half fragment go into the immediate offset
  constexpr int TR_LPR = ES == 2 ? 4 : 2;
  constexpr int TR_PITCH = BN * ES;
  constexpr int TR_KS_OFF = (16 / ES * 2) * TR_PITCH;
  constexpr int TR_R_OFF = (16 / TR_LPR) * TR_PITCH;
  if constexpr (!B_KC) {
    static_assert(B_KC || (TR_KS_OFF + TR_R_OFF < 65536 && TR_KS_OFF == B_BYTES / 2), "immediate offsets");
    const int i16 = lane & 15, ti = i16 / TR_LPR;
    const int n_sub = ((lane >> 4) & 1) * 16 + (i16 % TR_LPR) * (8 / ES);
    const int krow = (lane >> 5) * (16 / TR_LPR * 2) + ti;
    const int f = ES == 2 ? (ti & 3) << 2 : (ti & 7) << 1;
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
  u32x4_t af[2][FM], bf[2][FN];  // register sets of fragments: one per MFMA step, alternating
  u32x2_t bh[2][FN][2];          // row-major B: the two halves of a fragment as they come out of the transposing reads

  // 32 rows of a fragment are two 16-row groups: 2 KiB per fragment
  auto read_one = [&](auto set_c, auto r_c, auto jr_c, auto ks_c) {
    constexpr int SET = decltype(set_c)::value, R = decltype(r_c)::value;
    constexpr int JR = decltype(jr_c)::value, KS = decltype(ks_c)::value;
    if constexpr (R < FM) asm_ds_read16<R * 2048>(af[SET][R], a_addr[JR][KS]);
    else if constexpr (B_KC) asm_ds_read16<(R - FM) * 2048>(bf[SET][R - FM], b_addr[JR][KS]);
    else {  // K rows 16 KS .. of the slab sit in the group of parity KS / 2, at its local step KS % 2
      constexpr int J = (R - FM) / 2, HALF = (R - FM) % 2, ST = (2 * JR + KS / 2) % NST;
      asm_ds_read_tr<ES, (KS % 2) * TR_KS_OFF + HALF * TR_R_OFF>(bh[SET][J][HALF], b_addr[ST][J]);
    }
  };

  // One MFMA step: NMMA MFMAs on register set SET; after MFMA q the q-th memory instruction of the step:
  // first the NRD fragment reads of (ring position RJ, step RKS) into the other set, then this step's copies
  // (the A rows, the B rows or both of group c, parity CP, into buffer cst).
  auto step = [&](auto set_c, auto rj_c, auto rks_c, auto kind_c, auto cp_c, int cst, int c, uint64_t cmask) {
    constexpr int SET = decltype(set_c)::value;
    constexpr int KIND = decltype(kind_c)::value;   // copies of this step: 0 none, 1 A rows, 2 B rows, 3 both
    constexpr int NA = (KIND & 1) ? A_PW : 0, NB = (KIND & 2) ? B_PW : 0;
    constexpr int NOPS = NRD + NA + NB;
    constexpr int PER = (NOPS + NMMA - 1) / NMMA;
    static_assert(PER <= 2, "at most two memory instructions per MFMA");
    asm volatile("s_waitcnt lgkmcnt(0)");
    if constexpr (!B_KC) {
#pragma unroll
      for (int j = 0; j < FN; j++) {
        asm volatile("" : "+v"(bh[SET][j][0]), "+v"(bh[SET][j][1]));  // after the wait
        bf[SET][j] = u32x4_t{bh[SET][j][0][0], bh[SET][j][0][1], bh[SET][j][1][0], bh[SET][j][1][1]};
      }
    }
    if constexpr (NA > 0) copy_a_begin(cst);
    else if constexpr (NB > 0) copy_b_begin(cst);
    static_for<NMMA>([&](auto q_c) {
      constexpr int Q = decltype(q_c)::value;
      asm_mfma32<TYPES>(acc[Q / FN][Q % FN], bf[SET][Q % FN], af[SET][Q / FN]);
      static_for<PER>([&](auto o_c) {
        constexpr int OP = Q * PER + decltype(o_c)::value;
        if constexpr (OP < NRD) {
          read_one(std::integral_constant<int, SET ^ 1>{}, std::integral_constant<int, OP>{}, rj_c, rks_c);
        } else if constexpr (OP < NRD + NA) {
          copy_a(std::integral_constant<int, OP - NRD>{}, cp_c, c, cmask);
        } else if constexpr (OP < NOPS) {
          if constexpr (NA > 0 && OP == NRD + NA) copy_b_begin(cst);
          copy_b(std::integral_constant<int, OP - NRD - NA>{}, cp_c, c, cmask);
        }
      });
    });
  };

  const std::integral_constant<int, 0> no_copy{};
  const std::integral_constant<int, 1> is_a{};
  const std::integral_constant<int, 2> is_b{};
  const std::integral_constant<int, 3> a_and_b{};
  using I0 = std::integral_constant<int, 0>;
  using I1 = std::integral_constant<int, 1>;
  using I2 = std::integral_constant<int, 2>;
  using I3 = std::integral_constant<int, 3>;
  // lane mask of a copy as a scalar register pair: all ones while the group exists, zero past the end
  auto mask_if = [](bool on) -> uint64_t {
    const uint32_t w = (uint32_t)__builtin_amdgcn_readfirstlane(on ? -1 : 0);
    return ((uint64_t)w << 32) | w;
  };

  // ---- prologue: groups 0, 1, 2 whole and (EARLY_ODD: all of) the A rows of 3 ----
  static_for<EARLY_ODD ? 4 : 3>([&](auto c_c) {
    constexpr int C = decltype(c_c)::value;
    const uint64_t m = mask_if(C < nc);
    copy_a_begin(C);
    static_for<A_PW>([&](auto t) { copy_a(t, std::integral_constant<int, C & 1>{}, C, m); });
    copy_b_begin(C);
    static_for<B_PW>([&](auto t) { copy_b(t, std::integral_constant<int, C & 1>{}, C, m); });
  });
  if constexpr (!EARLY_ODD) {
    copy_a_begin(3);
    const uint64_t m3 = mask_if(3 < nc);
    static_for<A_PW>([&](auto t) { copy_a(t, I1{}, 3, m3); });
  }
  // slab 0 (groups 0 and 1) has landed; what was issued after it may still be on its way
  asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" : : "i"(EARLY_ODD ? 2 * NCP : NCP + A_PW) : "memory");
  static_for<NRD>([&](auto r) { read_one(I0{}, r, I0{}, I0{}); });

  // ---- one slab; JR = j % 5 at compile time ----
  auto slab = [&](auto jr_c, int j) {
    constexpr int JR = decltype(jr_c)::value;
    using NEXT = std::integral_constant<int, (JR + 1) % NST>;
    const int c3 = 2 * j + 3, c4 = 2 * j + 4, c5 = 2 * j + 5;
    const uint64_t m4 = mask_if(c4 < nc);
    if constexpr (EARLY_ODD) {
      step(I0{}, jr_c, I1{}, is_a, I0{}, (2 * JR + 4) % NST, c4, m4);
      step(I1{}, jr_c, I2{}, is_b, I0{}, (2 * JR + 4) % NST, c4, m4);
      step(I0{}, jr_c, I3{}, no_copy, I0{}, 0, 0, m4);
    } else {
      step(I0{}, jr_c, I1{}, is_b, I1{}, (2 * JR + 3) % NST, c3, mask_if(c3 < nc));
      step(I1{}, jr_c, I2{}, is_a, I0{}, (2 * JR + 4) % NST, c4, m4);
      step(I0{}, jr_c, I3{}, is_b, I0{}, (2 * JR + 4) % NST, c4, m4);
    }
    if (c4 < nc) {  // the copies of group 2j+4 may stay in flight
      if constexpr (NCP == 8) asm volatile("s_waitcnt vmcnt(8) lgkmcnt(0)\n\ts_barrier" ::: "memory");
      else asm volatile("s_waitcnt vmcnt(4) lgkmcnt(0)\n\ts_barrier" ::: "memory");
    } else {
      asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");
    }
    if constexpr (EARLY_ODD) step(I1{}, NEXT{}, I0{}, a_and_b, I1{}, (2 * JR + 5) % NST, c5, mask_if(c5 < nc));
    else step(I1{}, NEXT{}, I0{}, is_a, I1{}, (2 * JR + 5) % NST, c5, mask_if(c5 < nc));
  };

  const int nslab = nc / 2;
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
    asm_touch_acc<TYPES>(acc[Q / FN][Q % FN]);
  });

  static_assert(NW * epilogue_region_bytes<FN>() <= NST * STAGE_BYTES, "the epilogue reuses the operand buffers");
  __syncthreads();   // no wave reads operands any more and no copy is in flight
  store_accumulators_lds<TYPES, FM, FN, RAGGED>(g, acc, m0 + wm * WM, n0 + wn * WN, lane, lds + wave * epilogue_region_bytes<FN>());
}

}  // namespace gz
