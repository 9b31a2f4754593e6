/*
 * gz_oracle.c -- CPU restatement of gemm-zoo's reference GEMM.
 *
 * THIS FILE IS TEST INFRASTRUCTURE.  It is the checker the HIP kernels are
 * compared against; nothing in the shipped library links, loads or calls it.
 * Only the test-suite, the smoke check and the "cpu_baseline" leg of the
 * benchmark may load the shared object built from it.
 *
 * What it restates (paths are relative to the reference checkout):
 *
 *   - intel/utils/reference_kernel.hpp:12-28  (utils::detail::reference_gemm)
 *     twin: nvidia/kernels/naive_gemm.cuh:6-21
 *       one output element per work-item, sequential k from 0, accumulate in
 *       TOut, then  d = alpha*acc + beta*c.      -> oracle_literal_*()
 *
 *   - nvidia/kernels/generic_gemm.cuh:6-60  (nvidia::kernels::generic_gemm)
 *       inputs cast to float, float sum over k, then
 *       val = TOut(sum)*alpha; if (beta != 0) val += beta*c   (lines 53-58)
 *       evaluated in TOut arithmetic.            -> oracle_gemm()
 *
 *   - fp32 x fp32 -> fp32, the type of the reference's own ladder drivers (nvidia/bench/bench_naive.cu:9-17):
 *     the same loops with each product fused into the running sum (fmaf), which is what `acc += a * b`
 *     (nvidia/kernels/naive_gemm.cuh:16-19) compiles to under the reference's compilers' defaults.
 *
 *   - fp8 x fp8 -> fp16 (nvidia/bench/bench_cublaslt_e4m3.cu:6-21, bench_cublaslt_e5m2.cu:6-21: __nv_fp8_e4m3 /
 *     __nv_fp8_e5m2 inputs, __half output): the reference has no kernel of its own for these, only cuBLASLt and the
 *     generic checker, which "does all the compute in float" (nvidia/kernels/generic_gemm.cuh:10-13): the same
 *     oracle_gemm() loop on decoded inputs with the fp16 epilogue.  The two formats are the OCP 8-bit floats
 *     (OCP 8-bit Floating Point Specification v1.0): e4m3 = 1-4-3 bits, bias 7, no infinities, S.1111.111 NaN,
 *     largest finite 448; e5m2 = 1-5-2 bits, bias 15, IEEE-style infinities and NaNs.   -> oracle_fp8_*()
 *
 *   - the 16-bit accumulators of intel/kernels/xe_gemm_bf16_bf16_bf16_m8k16.hpp:88-107 (bf16 C operand of every
 *     DPAS, bf16 epilogue) and nvidia/kernels/sm_80/fp16_mma_gemm.cuh:179,279-290 (fp16 C operand of every
 *     mma.sync.m16n8k8, mul.f16x2 / fma.rn.f16x2 epilogue) as the bundles *_ACC16: chunks of 16 / 8 k, fp32 inside
 *     a chunk, the running sum rounded to 16 bits after every chunk (see store_acc16 and the comment above it).
 *     What the two devices do inside one instruction is not published and the reference holds no output of
 *     these kernels: the model is pinned as arithmetic (below), its agreement with either device is
 *     PARITY UNPINNED.
 *
 *   - layouts: the reference only knows row-major operands; column-major A/B
 *     is the generalisation  A(i,p) = rowmajor ? a[i*K+p] : a[p*M+i].
 *
 *   - intel/test/utils.hpp:27-45 (populate_with_random): a counter based
 *     Philox4x32-10 stream keyed by (seed, element_id).  The reference's exact
 *     streams come from oneMath / cuRAND and cannot be reproduced; only the
 *     construction (one engine per element, keyed by seed and element index)
 *     is followed.                               -> oracle_fill_*()
 *
 * Pinning (see tests/test_oracle_*.py):
 *   oracle_literal_*      closed forms (all-ones, identity, single-nonzero
 *                         probes, extreme int8), brute force vs Python ints.
 *   oracle_gemm           bit-equal to oracle_literal_* on row-major inputs
 *                         for s8->s32 and for integer-valued float inputs;
 *                         fp64 truth within fp32 accumulation bounds; layout
 *                         probes; beta==0 never reads C.
 *   fp32 bundle           exact rational arithmetic rounded once per step (distinguishes the fused sum from
 *                         multiply-then-add), integer-valued inputs, fp64 truth.
 *   fp8 decode / encode   every one of the 256 codes of both formats against torch.float8_e4m3fn / float8_e5m2
 *                         (an independent implementation), the specification's table of extreme values,
 *                         encode(decode(code)) == code, ties-to-even and saturation known answers; the GEMM
 *                         on fp8 inputs against exact integer arithmetic (every product and partial sum of
 *                         small codes is exact) and fp64 truth.
 *   *_ACC16 bundles       closed forms that separate a 16-bit running sum from an fp32 one and one chunk length
 *                         from another (K ones stop growing at 4096 for bf16 / 16, at 16384 for fp16 / 8), an
 *                         independent model in numpy (float32 adds, numpy float16 / torch bfloat16 roundings),
 *                         oracle_f64_to_f16 against numpy on every fp16 value, its midpoints and neighbours,
 *                         oracle_fma_f16 against exact rational arithmetic incl. a product on a rounding tie
 *                         that a tiny addend must break (fails any two-step multiply-add).
 *   bf16/fp16 converters  closed-form RNE known answers, exhaustive 2^16
 *                         round trips, numpy float16 / torch bfloat16.
 *   philox4x32_10         Random123 known-answer vectors.
 *   normal/uniform fills  moments + distribution bounds (self-defined stream:
 *                         "parity unpinned" with respect to the reference's
 *                         cuRAND / oneMath streams, which nothing in the
 *                         reference records).
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define ORACLE_API __attribute__((visibility("default")))

enum { OR_S8S8S32 = 0, OR_BF16BF16F32 = 1, OR_BF16BF16BF16 = 2, OR_F16F16F16 = 3, OR_F32F32F32 = 4,
       OR_E4M3E4M3F16 = 5, OR_E5M2E5M2F16 = 6, OR_BF16BF16BF16_ACC16 = 7, OR_F16F16F16_ACC16 = 8, OR_NUM_TYPES = 9 };
enum { OR_ROW = 0, OR_COL = 1 };

/* ------------------------------------------------------------------------ */
/* 16-bit float conversions (round-to-nearest-even)                          */
/* ------------------------------------------------------------------------ */
static inline uint32_t f32_bits(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline float bits_f32(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }

ORACLE_API float oracle_bf16_to_f32(uint16_t h) { return bits_f32((uint32_t)h << 16); }

ORACLE_API uint16_t oracle_f32_to_bf16(float f) {
  uint32_t u = f32_bits(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u); /* quiet NaN */
  uint32_t lsb = (u >> 16) & 1u;
  u += 0x7fffu + lsb;
  return (uint16_t)(u >> 16);
}

ORACLE_API float oracle_f16_to_f32(uint16_t h) {
  uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  uint32_t exp = (h >> 10) & 0x1fu;
  uint32_t man = h & 0x3ffu;
  if (exp == 0) {
    if (man == 0) return bits_f32(sign);
    /* subnormal: value = man * 2^-24 */
    float v = (float)man * 5.9604644775390625e-8f;
    return bits_f32(f32_bits(v) | sign);
  }
  if (exp == 31) return bits_f32(sign | 0x7f800000u | (man << 13));
  return bits_f32(sign | ((exp + 112u) << 23) | (man << 13));
}

ORACLE_API uint16_t oracle_f32_to_f16(float f) {
  uint32_t u = f32_bits(f);
  uint16_t sign = (uint16_t)((u >> 16) & 0x8000u);
  uint32_t a = u & 0x7fffffffu;
  if (a > 0x7f800000u) return (uint16_t)(sign | 0x7e00u | ((a >> 13) & 0x3ffu)); /* NaN */
  if (a >= 0x477ff000u) return (uint16_t)(sign | 0x7c00u); /* >= 65520 rounds to inf */
  if (a < 0x33000000u) {                                  /* < 2^-25 : rounds to 0   */
    /* exactly 2^-25 ties to even (0); anything larger than 2^-25 goes up */
    return sign;
  }
  int32_t e = (int32_t)(a >> 23) - 127;
  uint32_t m = (a & 0x7fffffu) | 0x800000u; /* 24-bit significand */
  int shift;                                /* bits dropped from m */
  uint32_t base;
  if (e < -14) { /* subnormal half: unit is 2^-24 */
    shift = 13 + (-14 - e);
    base = 0;
  } else {
    shift = 13;
    base = (uint32_t)(e + 15) << 10;
    m &= 0x7fffffu;
  }
  uint32_t q = m >> shift;
  uint32_t rem = m & ((1u << shift) - 1u);
  uint32_t half = 1u << (shift - 1);
  if (rem > half || (rem == half && (q & 1u))) q++;
  return (uint16_t)(sign | (base + q)); /* carry into exponent is intended */
}

/* ------------------------------------------------------------------------ */
/* OCP 8-bit floats, from the format definition:                             */
/*   normal     (-1)^s * 2^(E - bias) * (1 + m / 2^MAN)      1 <= E          */
/*   subnormal  (-1)^s * 2^(1 - bias) * (m / 2^MAN)          E == 0          */
/* e4m3 (bias 7): E == 15 is an ordinary exponent, except S.1111.111 = NaN.  */
/* e5m2 (bias 15): E == 31 is infinity (m == 0) or NaN.                      */
/* ------------------------------------------------------------------------ */
ORACLE_API float oracle_fp8_to_f32(int e5m2, uint8_t code) {
  const int man_bits = e5m2 ? 2 : 3, bias = e5m2 ? 15 : 7;
  const int sign = code >> 7, E = (code & 0x7f) >> man_bits, m = code & ((1 << man_bits) - 1);
  float mag;
  if (e5m2 && E == 31) mag = m ? NAN : INFINITY;
  else if (!e5m2 && E == 15 && m == 7) mag = NAN;
  else if (E == 0) mag = ldexpf((float)m, 1 - bias - man_bits);
  else mag = ldexpf((float)((1 << man_bits) + m), E - bias - man_bits);
  return sign ? -mag : mag;
}

/* Nearest finite code, ties to the code with an even mantissa, beyond the largest finite value: that value
 * (the saturating conversion; what the device fill uses).  Found by search over the 2^7 magnitudes, which is
 * slow and obviously right.                                                                                */
ORACLE_API uint8_t oracle_f32_to_fp8(int e5m2, float f) {
  const uint8_t sign = signbit(f) ? 0x80 : 0;
  if (isnan(f)) return (uint8_t)(sign | 0x7f);
  const uint8_t max_code = e5m2 ? 0x7b : 0x7e;
  const double a = fabs((double)f);
  if (isinf(f) || a >= (double)oracle_fp8_to_f32(e5m2, max_code)) return (uint8_t)(sign | max_code);
  uint8_t best = 0;
  double best_err = a; /* distance to code 0 */
  for (int c = 1; c <= max_code; c++) {
    const double err = fabs(a - (double)oracle_fp8_to_f32(e5m2, (uint8_t)c));
    if (err < best_err || (err == best_err && (c & 1) == 0)) { best = (uint8_t)c; best_err = err; }
  }
  return (uint8_t)(sign | best);
}

static inline int is_fp8(int types) { return types == OR_E4M3E4M3F16 || types == OR_E5M2E5M2F16; }

static inline int is_acc16(int types) { return types == OR_BF16BF16BF16_ACC16 || types == OR_F16F16F16_ACC16; }
static inline int out_is_bf16(int types) { return types == OR_BF16BF16BF16 || types == OR_BF16BF16BF16_ACC16; }
static inline int in_is_f16(int types) { return types == OR_F16F16F16 || types == OR_F16F16F16_ACC16; }

static inline float round_to(int types, float v) {
  if (out_is_bf16(types)) return oracle_bf16_to_f32(oracle_f32_to_bf16(v));
  if (in_is_f16(types) || is_fp8(types)) return oracle_f16_to_f32(oracle_f32_to_f16(v));
  return v;
}

/* ------------------------------------------------------------------------ */
/* The reference kernels' 16-bit accumulators (opt-in bundles *_ACC16).      */
/*   intel/kernels/xe_gemm_bf16_bf16_bf16_m8k16.hpp:88-97: two DPAS per k-tile of 32, 16 k each, with the        */
/*     SPIRV_MatrixCBf16 flag: the accumulator that goes in and comes out of every instruction is bf16.          */
/*   nvidia/kernels/sm_80/fp16_mma_gemm.cuh:179: mma.sync.m16n8k8 ... f16.f16.f16.f16, 8 k each, fp16 C and D.   */
/* How either device sums inside one instruction is not published.  The model: K is cut into chunks of 16        */
/* (bf16) / 8 (fp16) consecutive k; a chunk's exact products are added in k order in fp32 from zero; the         */
/* running sum becomes T(fp32(sum + chunk)).  A last, shorter chunk is a chunk like any other.                   */
/* Epilogues: bf16  d = T(T(alpha*acc) + T(beta*c))  (xe_gemm_bf16_bf16_bf16_m8k16.hpp:104-107: the operators    */
/*   of sycl's bfloat16 compute in float and round the result), the generic epilogue on an already-bf16 sum;     */
/*   fp16  d = fma.rn.f16(alpha, acc, mul.f16(beta, c))  (fp16_mma_gemm.cuh:279-290): one rounding for the fused */
/*   multiply-add.  beta == 0: c is not read, the addend is +0.                                                  */
/* ------------------------------------------------------------------------ */
static inline int acc16_chunk(int types) { return types == OR_BF16BF16BF16_ACC16 ? 16 : 8; }

/* double -> fp16, round to nearest even, from the value itself (no intermediate float) */
ORACLE_API uint16_t oracle_f64_to_f16(double v) {
  uint64_t bits; memcpy(&bits, &v, 8);
  const uint16_t sign = (uint16_t)((bits >> 48) & 0x8000u);
  if (isnan(v)) return (uint16_t)(sign | 0x7e00u);
  const double a = fabs(v);
  if (a >= 65520.0) return (uint16_t)(sign | 0x7c00u); /* halfway between 65504 and 2^16 rounds to even = infinity */
  if (a == 0.0) return sign;
  int e; (void)frexp(a, &e);          /* a = m 2^e, 0.5 <= m < 1: leading bit 2^(e-1) */
  int E = e - 1;
  if (E < -14) E = -14;               /* subnormals share the smallest normal's spacing */
  const double q = rint(ldexp(a, 10 - E)); /* a in units of 2^(E-10): exact scaling, then nearest-even (default mode) */
  /* normal: q in [1024, 2048] holds the implicit bit, so ((E+14) << 10) + q; subnormal: E = -14, the code is q;
   * a carry to 2048 lands in the next binade either way */
  return (uint16_t)(sign | (uint16_t)(((uint32_t)(E + 14) << 10) + (uint32_t)q));
}

/* fma.rn.f16: a*b + c rounded once.  a, b, c hold fp16 values, so a*b is exact in double; the sum is exact in double
 * unless the addends are very far apart, and then the low part (TwoSum) only has to break a tie */
ORACLE_API uint16_t oracle_fma_f16(float a, float b, float c) {
  const double p = (double)a * (double)b;
  double s = p + (double)c;
  if (isfinite(s)) {
    const double bb = s - p;
    const double err = (p - (s - bb)) + ((double)c - bb);
    if (err > 0) s = nextafter(s, INFINITY);
    else if (err < 0) s = nextafter(s, -INFINITY);
  }
  return oracle_f64_to_f16(s);
}

/* epilogue of the *_ACC16 bundles on a running sum `acc` that already holds a value of the output type */
static inline void store_acc16(int types, void* D, const void* C, size_t idx, float acc, float alpha, float beta) {
  uint16_t* d = (uint16_t*)D;
  const uint16_t* c = (const uint16_t*)C;
  if (types == OR_BF16BF16BF16_ACC16) {
    float val = round_to(types, acc * alpha);
    if (beta != 0.0f) val = round_to(types, val + round_to(types, beta * oracle_bf16_to_f32(c[idx])));
    d[idx] = oracle_f32_to_bf16(val);
  } else {
    const float bc = beta != 0.0f ? round_to(types, beta * oracle_f16_to_f32(c[idx])) : 0.0f;
    d[idx] = oracle_fma_f16(alpha, acc, bc);
  }
}

/* ------------------------------------------------------------------------ */
/* Literal loops (intel/utils/reference_kernel.hpp:16-28)                    */
/* row-major A (m x k), row-major B (k x n), row-major C/D, C always read.   */
/* ------------------------------------------------------------------------ */
ORACLE_API void oracle_literal_s8s32(const int8_t* a, const int8_t* b, const int32_t* c, int32_t* d,
                                     size_t m, size_t n, size_t k, int32_t alpha, int32_t beta) {
  for (size_t gid = 0; gid < m * n; gid++) {
    const size_t output_row = gid / n;
    const size_t output_col = gid % n;
    uint32_t acc = 0; /* two's-complement int32 arithmetic */
    for (size_t i = 0; i < k; i++) {
      acc += (uint32_t)((int32_t)a[output_row * k + i] * (int32_t)b[i * n + output_col]);
    }
    acc = (uint32_t)alpha * acc + (uint32_t)beta * (uint32_t)c[output_row * n + output_col];
    d[output_row * n + output_col] = (int32_t)acc;
  }
}

/* TOut = float instantiation; inputs already widened to float by the caller
 * (the widening of bf16/fp16 to fp32 is exact).                              */
ORACLE_API void oracle_literal_f32(const float* a, const float* b, const float* c, float* d,
                                   size_t m, size_t n, size_t k, float alpha, float beta) {
  for (size_t gid = 0; gid < m * n; gid++) {
    const size_t output_row = gid / n;
    const size_t output_col = gid % n;
    float acc = 0.0f;
    for (size_t i = 0; i < k; i++) {
      acc += a[output_row * k + i] * b[i * n + output_col];
    }
    acc = alpha * acc + beta * c[output_row * n + output_col];
    d[output_row * n + output_col] = acc;
  }
}

/* ------------------------------------------------------------------------ */
/* General oracle: any layout, fp32 (or int32) sequential-k accumulate,      */
/* generic_gemm epilogue (nvidia/kernels/generic_gemm.cuh:53-58).            */
/* The j-inner loop order keeps each output's own summation order sequential */
/* in k, exactly like the literal loop, while letting the compiler vectorise */
/* across outputs.                                                           */
/* ------------------------------------------------------------------------ */
static size_t in_size(int types) {
  return (types == OR_S8S8S32 || types == OR_E4M3E4M3F16 || types == OR_E5M2E5M2F16) ? 1 : types == OR_F32F32F32 ? 4 : 2;
}
static size_t out_size(int types) {
  return (types == OR_S8S8S32 || types == OR_BF16BF16F32 || types == OR_F32F32F32) ? 4 : 2;
}

static float load_in_f32(int types, const void* p, size_t idx) {
  if (types == OR_F32F32F32) return ((const float*)p)[idx];
  if (types == OR_E4M3E4M3F16) return oracle_fp8_to_f32(0, ((const uint8_t*)p)[idx]);
  if (types == OR_E5M2E5M2F16) return oracle_fp8_to_f32(1, ((const uint8_t*)p)[idx]);
  const uint16_t* h = (const uint16_t*)p;
  return in_is_f16(types) ? oracle_f16_to_f32(h[idx]) : oracle_bf16_to_f32(h[idx]);
}

static float load_out_f32(int types, const void* p, size_t idx) {
  if (types == OR_BF16BF16F32 || types == OR_F32F32F32) return ((const float*)p)[idx];
  if (out_is_bf16(types)) return oracle_bf16_to_f32(((const uint16_t*)p)[idx]);
  return oracle_f16_to_f32(((const uint16_t*)p)[idx]);
}

static void store_out_f32(int types, void* p, size_t idx, float v) {
  if (types == OR_BF16BF16F32 || types == OR_F32F32F32) ((float*)p)[idx] = v;
  else if (out_is_bf16(types)) ((uint16_t*)p)[idx] = oracle_f32_to_bf16(v);
  else ((uint16_t*)p)[idx] = oracle_f32_to_f16(v);
}

/* Computes rows [row0, row1) of D.  Returns 0 on success. */
ORACLE_API int oracle_gemm_rows(int types, const void* A, const void* B, const void* C, void* D,
                                int64_t M, int64_t N, int64_t K, int layoutA, int layoutB,
                                double alpha_d, double beta_d, int64_t row0, int64_t row1,
                                int threads) {
  if (types < 0 || types >= OR_NUM_TYPES || M < 0 || N < 0 || K < 0) return 1;
  if (row0 < 0 || row1 > M || row0 > row1) return 1;
  if (M == 0 || N == 0) return 0;
#ifdef _OPENMP
  if (threads <= 0) threads = omp_get_max_threads();
#else
  threads = 1;
#endif

  if (types == OR_S8S8S32) {
    const int8_t* a = (const int8_t*)A;
    const int8_t* b = (const int8_t*)B;
    const int32_t* c = (const int32_t*)C;
    int32_t* d = (int32_t*)D;
    const uint32_t alpha = (uint32_t)(int32_t)alpha_d, beta = (uint32_t)(int32_t)beta_d;
    /* pure data movement: B as row-major K x N so the j loop is contiguous */
    int8_t* bt = NULL;
    if (layoutB == OR_COL && K > 0) {
      bt = (int8_t*)malloc((size_t)K * N);
      if (!bt) return 2;
#pragma omp parallel for num_threads(threads) schedule(static)
      for (int64_t p = 0; p < K; p++)
        for (int64_t j = 0; j < N; j++) bt[p * N + j] = b[j * K + p];
      b = bt;
    }
#pragma omp parallel num_threads(threads)
    {
      uint32_t* acc = (uint32_t*)malloc(sizeof(uint32_t) * (size_t)N);
#pragma omp for schedule(dynamic, 4)
      for (int64_t i = row0; i < row1; i++) {
        for (int64_t j = 0; j < N; j++) acc[j] = 0;
        for (int64_t p = 0; p < K; p++) {
          const int32_t av = layoutA == OR_ROW ? a[i * K + p] : a[p * M + i];
          const int8_t* brow = b + p * N;
          for (int64_t j = 0; j < N; j++) acc[j] += (uint32_t)(av * (int32_t)brow[j]);
        }
        for (int64_t j = 0; j < N; j++) {
          uint32_t v = alpha * acc[j];
          if (beta != 0) v += beta * (uint32_t)c[i * N + j];
          d[i * N + j] = (int32_t)v;
        }
      }
      free(acc);
    }
    free(bt);
    return 0;
  }

  /* float paths */
  const float alpha = round_to(types, (float)alpha_d);
  const float beta = round_to(types, (float)beta_d);
  float* bf = K > 0 ? (float*)malloc(sizeof(float) * (size_t)K * N) : NULL;
  if (K > 0 && !bf) return 2;
#pragma omp parallel for num_threads(threads) schedule(static)
  for (int64_t p = 0; p < K; p++)
    for (int64_t j = 0; j < N; j++)
      bf[p * N + j] = load_in_f32(types, B, layoutB == OR_ROW ? (size_t)(p * N + j) : (size_t)(j * K + p));

#pragma omp parallel num_threads(threads)
  {
    float* acc = (float*)malloc(sizeof(float) * (size_t)N * 2);
    float* part = acc + N;
#pragma omp for schedule(dynamic, 4)
    for (int64_t i = row0; i < row1; i++) {
      for (int64_t j = 0; j < N; j++) acc[j] = 0.0f, part[j] = 0.0f;
      for (int64_t p = 0; p < K; p++) {
        const float av = load_in_f32(types, A, layoutA == OR_ROW ? (size_t)(i * K + p) : (size_t)(p * M + i));
        const float* brow = bf + p * N;
        if (is_acc16(types)) {
          /* 16-bit running sum: the chunk's products in fp32 from zero, folded at the chunk's last k */
          for (int64_t j = 0; j < N; j++) part[j] = part[j] + av * brow[j];
          if ((p + 1) % acc16_chunk(types) == 0 || p + 1 == K)
            for (int64_t j = 0; j < N; j++) acc[j] = round_to(types, acc[j] + part[j]), part[j] = 0.0f;
        } else if (types == OR_F32F32F32) {
          /* fp32 inputs: the product is fused into the sum, which is what `acc += a * b` of the reference
           * kernels (nvidia/kernels/naive_gemm.cuh:16-19) compiles to under nvcc's and icpx's defaults */
          for (int64_t j = 0; j < N; j++) acc[j] = __builtin_fmaf(av, brow[j], acc[j]);
        } else {
          /* a*b is exact in fp32 for 16-bit inputs; one rounding per add */
          for (int64_t j = 0; j < N; j++) acc[j] = acc[j] + av * brow[j];
        }
      }
      if (is_acc16(types)) {
        for (int64_t j = 0; j < N; j++) store_acc16(types, D, C, (size_t)(i * N + j), acc[j], alpha, beta);
        continue;
      }
      for (int64_t j = 0; j < N; j++) {
        /* generic_gemm.cuh:53-58, every operation rounded to TOut */
        float val = round_to(types, acc[j]);
        val = round_to(types, val * alpha);
        if (beta != 0.0f) {
          float bc = round_to(types, beta * load_out_f32(types, C, (size_t)(i * N + j)));
          val = round_to(types, val + bc);
        }
        store_out_f32(types, D, (size_t)(i * N + j), val);
      }
    }
    free(acc);
  }
  free(bf);
  return 0;
}

ORACLE_API int oracle_gemm(int types, const void* A, const void* B, const void* C, void* D,
                           int64_t M, int64_t N, int64_t K, int layoutA, int layoutB,
                           double alpha, double beta, int threads) {
  return oracle_gemm_rows(types, A, B, C, D, M, N, K, layoutA, layoutB, alpha, beta, 0, M, threads);
}

/* The literal one-work-item-per-output loop for any type pair and layout,
 * parallelised as the reference parallelises it (one output element per
 * work-item, reference_kernel.hpp:36-37 -> omp over the flattened index).
 * Used as the CPU baseline timed beside the GPU number; accumulates in fp32
 * (int32) and applies the same epilogue as oracle_gemm.                     */
ORACLE_API int oracle_gemm_naive_rows(int types, const void* A, const void* B, const void* C, void* D,
                                      int64_t M, int64_t N, int64_t K, int layoutA, int layoutB,
                                      double alpha_d, double beta_d, int64_t row0, int64_t row1,
                                      int threads) {
  if (types < 0 || types >= OR_NUM_TYPES || M < 0 || N < 0 || K < 0) return 1;
  if (row0 < 0 || row1 > M || row0 > row1) return 1;
  if (N == 0) return 0;
#ifdef _OPENMP
  if (threads <= 0) threads = omp_get_max_threads();
#else
  threads = 1;
#endif
  const float alpha = round_to(types, (float)alpha_d);
  const float beta = round_to(types, (float)beta_d);
  const uint32_t ialpha = (uint32_t)(int32_t)alpha_d, ibeta = (uint32_t)(int32_t)beta_d;
#pragma omp parallel for num_threads(threads) schedule(static)
  for (int64_t gid = row0 * N; gid < row1 * N; gid++) {
    const int64_t i = gid / N, j = gid % N;
    if (types == OR_S8S8S32) {
      const int8_t* a = (const int8_t*)A;
      const int8_t* b = (const int8_t*)B;
      uint32_t acc = 0;
      for (int64_t p = 0; p < K; p++) {
        int32_t av = layoutA == OR_ROW ? a[i * K + p] : a[p * M + i];
        int32_t bv = layoutB == OR_ROW ? b[p * N + j] : b[j * K + p];
        acc += (uint32_t)(av * bv);
      }
      uint32_t v = ialpha * acc;
      if (ibeta != 0) v += ibeta * (uint32_t)((const int32_t*)C)[gid];
      ((int32_t*)D)[gid] = (int32_t)v;
    } else {
      float acc = 0.0f, part = 0.0f;
      for (int64_t p = 0; p < K; p++) {
        float av = load_in_f32(types, A, layoutA == OR_ROW ? (size_t)(i * K + p) : (size_t)(p * M + i));
        float bv = load_in_f32(types, B, layoutB == OR_ROW ? (size_t)(p * N + j) : (size_t)(j * K + p));
        if (is_acc16(types)) {
          part = part + av * bv;
          if ((p + 1) % acc16_chunk(types) == 0 || p + 1 == K) acc = round_to(types, acc + part), part = 0.0f;
        } else {
          acc = types == OR_F32F32F32 ? __builtin_fmaf(av, bv, acc) : acc + av * bv;
        }
      }
      if (is_acc16(types)) {
        store_acc16(types, D, C, (size_t)gid, acc, alpha, beta);
        continue;
      }
      float val = round_to(types, acc);
      val = round_to(types, val * alpha);
      if (beta != 0.0f) {
        float bc = round_to(types, beta * load_out_f32(types, C, (size_t)gid));
        val = round_to(types, val + bc);
      }
      store_out_f32(types, D, (size_t)gid, val);
    }
  }
  return 0;
}

/* fp64-accumulated product (no epilogue rounding): truth for tolerance tests.
 * out[i*N+j] = alpha * sum_p A(i,p) B(p,j) + beta * C(i,j), all in double.
 * absout (optional) receives sum_p |A(i,p)| |B(p,j)| for error bounds.       */
ORACLE_API int oracle_gemm_f64(int types, const void* A, const void* B, const void* C, double* out,
                               double* absout, int64_t M, int64_t N, int64_t K, int layoutA,
                               int layoutB, double alpha, double beta, int64_t row0, int64_t row1,
                               int threads) {
  if (types < 1 || types >= OR_NUM_TYPES) return 1;
#ifdef _OPENMP
  if (threads <= 0) threads = omp_get_max_threads();
#else
  threads = 1;
#endif
  double* bf = (double*)malloc(sizeof(double) * (size_t)(K > 0 ? K : 1) * N);
  if (!bf) return 2;
  for (int64_t p = 0; p < K; p++)
    for (int64_t j = 0; j < N; j++)
      bf[p * N + j] = load_in_f32(types, B, layoutB == OR_ROW ? (size_t)(p * N + j) : (size_t)(j * K + p));
#pragma omp parallel num_threads(threads)
  {
    double* acc = (double*)malloc(sizeof(double) * (size_t)N * 2);
    double* aac = acc + N;
#pragma omp for schedule(dynamic, 4)
    for (int64_t i = row0; i < row1; i++) {
      for (int64_t j = 0; j < N; j++) acc[j] = 0.0, aac[j] = 0.0;
      for (int64_t p = 0; p < K; p++) {
        const double av = load_in_f32(types, A, layoutA == OR_ROW ? (size_t)(i * K + p) : (size_t)(p * M + i));
        const double* brow = bf + p * N;
        for (int64_t j = 0; j < N; j++) {
          acc[j] += av * brow[j];
          aac[j] += fabs(av * brow[j]);
        }
      }
      for (int64_t j = 0; j < N; j++) {
        double v = alpha * acc[j];
        if (beta != 0.0) v += beta * (double)load_out_f32(types, C, (size_t)(i * N + j));
        out[(i - row0) * N + j] = v;
        if (absout) absout[(i - row0) * N + j] = aac[j];
      }
    }
    free(acc);
  }
  free(bf);
  return 0;
}

/* ------------------------------------------------------------------------ */
/* Philox4x32-10 (Salmon et al., SC'11), counter = element index, key = seed */
/* ------------------------------------------------------------------------ */
ORACLE_API void oracle_philox4x32_10(const uint32_t ctr_in[4], const uint32_t key_in[2], uint32_t out[4]) {
  uint32_t c0 = ctr_in[0], c1 = ctr_in[1], c2 = ctr_in[2], c3 = ctr_in[3];
  uint32_t k0 = key_in[0], k1 = key_in[1];
  for (int r = 0; r < 10; r++) {
    uint64_t p0 = (uint64_t)0xD2511F53u * c0;
    uint64_t p1 = (uint64_t)0xCD9E8D57u * c2;
    uint32_t n0 = (uint32_t)(p1 >> 32) ^ c1 ^ k0;
    uint32_t n1 = (uint32_t)p1;
    uint32_t n2 = (uint32_t)(p0 >> 32) ^ c3 ^ k1;
    uint32_t n3 = (uint32_t)p0;
    c0 = n0; c1 = n1; c2 = n2; c3 = n3;
    k0 += 0x9E3779B9u;
    k1 += 0xBB67AE85u;
  }
  out[0] = c0; out[1] = c1; out[2] = c2; out[3] = c3;
}

static inline void philox_elem(uint64_t seed, uint64_t idx, uint32_t out[4]) {
  uint32_t ctr[4] = {(uint32_t)idx, (uint32_t)(idx >> 32), 0u, 0u};
  uint32_t key[2] = {(uint32_t)seed, (uint32_t)(seed >> 32)};
  oracle_philox4x32_10(ctr, key, out);
}

/* --- transcendental-free-of-libm helpers: only IEEE-exact operations ------ *
 * (+, *, /, sqrt, fma), so that any IEEE implementation that evaluates the  *
 * same expression tree produces the same bits.                              */
static inline float fma_(float a, float b, float c) { return __builtin_fmaf(a, b, c); }

/* natural log of x in (0, 1]; |rel err| ~ 1e-7 */
static float det_logf(float x) {
  uint32_t u = f32_bits(x);
  int32_t e = (int32_t)(u >> 23) - 127;
  uint32_t mant = (u & 0x007fffffu) | 0x3f800000u; /* m in [1,2) */
  float m = bits_f32(mant);
  if (m > 1.41421356f) { m = m * 0.5f; e += 1; }   /* m in (0.707, 1.414] */
  float s = (m - 1.0f) / (m + 1.0f);
  float s2 = s * s;
  float p = 0.0909090909f;            /* 1/11 */
  p = fma_(p, s2, 0.1111111111f);     /* 1/9  */
  p = fma_(p, s2, 0.1428571429f);     /* 1/7  */
  p = fma_(p, s2, 0.2f);              /* 1/5  */
  p = fma_(p, s2, 0.3333333333f);     /* 1/3  */
  p = fma_(p, s2, 1.0f);
  float lm = (s + s) * p;
  return fma_((float)e, 0.693147180559945f, lm);
}

/* sin and cos of 2*pi*u for u in [0,1); |abs err| ~ 1e-7 */
static void det_sincos2pi(float u, float* sn, float* cs) {
  float t = u * 8.0f;                 /* exact */
  int oct = (int)t;                   /* 0..7 */
  float r = t - (float)oct;           /* exact, in [0,1) */
  if (oct & 1) r = 1.0f - r;          /* reflect odd octants: exact */
  float x = r * 0.785398163397448f;   /* angle in [0, pi/4] */
  float x2 = x * x;
  float sp = 2.7557319224e-6f;        /*  1/9! */
  sp = fma_(sp, x2, -1.9841269841e-4f);
  sp = fma_(sp, x2, 8.3333333333e-3f);
  sp = fma_(sp, x2, -1.6666666667e-1f);
  sp = fma_(sp, x2, 1.0f);
  float s = x * sp;
  float cp = 2.4801587302e-5f;        /*  1/8! */
  cp = fma_(cp, x2, -1.3888888889e-3f);
  cp = fma_(cp, x2, 4.1666666667e-2f);
  cp = fma_(cp, x2, -0.5f);
  cp = fma_(cp, x2, 1.0f);
  float c = cp;
  /* octant fix-up: angle = oct*pi/4 + (odd ? pi/4 - x : x) */
  float so, co;
  switch ((oct + 1) >> 1 & 3) {       /* nearest multiple of pi/2 */
    case 0: so = s; co = c; break;
    case 1: so = c; co = s; break;
    case 2: so = s; co = c; break;
    default: so = c; co = s; break;
  }
  /* signs by octant */
  static const signed char ssign[8] = {1, 1, 1, 1, -1, -1, -1, -1};
  static const signed char csign[8] = {1, 1, -1, -1, -1, -1, 1, 1};
  *sn = ssign[oct] > 0 ? so : -so;
  *cs = csign[oct] > 0 ? co : -co;
}

static inline float uniform01_open(uint32_t w) { /* (0,1]: (w>>8 + 1) * 2^-24, exact */
  return (float)((w >> 8) + 1u) * 5.9604644775390625e-8f;
}
static inline float uniform01(uint32_t w) {      /* [0,1): (w>>8) * 2^-24, exact */
  return (float)(w >> 8) * 5.9604644775390625e-8f;
}

ORACLE_API float oracle_normal_from_words(uint32_t w0, uint32_t w1) {
  float u1 = uniform01_open(w0);
  float u2 = uniform01(w1);
  float rad = __builtin_sqrtf(-2.0f * det_logf(u1));
  float sn, cs;
  det_sincos2pi(u2, &sn, &cs);
  (void)sn;
  return rad * cs;
}

/* kind: 0 = int8 uniform [-128,127] (low byte of word 0)
 *       1 = N(0,1)*scale      2 = U(-1,1)*scale      3 = integers {-1,0,1}
 *           (kind 3 mirrors intel/test/utils.hpp:35-41: uniform(-2,2)
 *            truncated toward zero, so every partial sum is exact)
 * dtype: 0 = int8, 1 = bf16, 2 = fp16, 3 = fp32, 4 = int32, 5 = fp8 e4m3, 6 = fp8 e5m2 (saturating) */
static float fill_value(int kind, float scale, uint64_t seed, uint64_t idx) {
  uint32_t w[4];
  philox_elem(seed, idx, w);
  switch (kind) {
    case 0: return (float)(int8_t)(w[0] & 0xffu);
    case 1: return oracle_normal_from_words(w[0], w[1]) * scale;
    case 2: return fma_(uniform01(w[0]), 2.0f, -1.0f) * scale;
    default: return (float)(int32_t)fma_(uniform01(w[0]), 4.0f, -2.0f);
  }
}

ORACLE_API int oracle_fill(void* dst, int64_t count, int dtype, int kind, float scale, uint64_t seed,
                           int threads) {
  if (count < 0 || dtype < 0 || dtype > 6 || kind < 0 || kind > 3) return 1;
#ifdef _OPENMP
  if (threads <= 0) threads = omp_get_max_threads();
#else
  threads = 1;
#endif
#pragma omp parallel for num_threads(threads) schedule(static)
  for (int64_t i = 0; i < count; i++) {
    float v = fill_value(kind, scale, seed, (uint64_t)i);
    switch (dtype) {
      case 5: ((uint8_t*)dst)[i] = oracle_f32_to_fp8(0, v); break;
      case 6: ((uint8_t*)dst)[i] = oracle_f32_to_fp8(1, v); break;
      case 0: ((int8_t*)dst)[i] = (int8_t)v; break;
      case 1: ((uint16_t*)dst)[i] = oracle_f32_to_bf16(v); break;
      case 2: ((uint16_t*)dst)[i] = oracle_f32_to_f16(v); break;
      case 3: ((float*)dst)[i] = v; break;
      default: ((int32_t*)dst)[i] = (int32_t)v; break;
    }
  }
  return 0;
}

ORACLE_API int oracle_num_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}

ORACLE_API size_t oracle_in_size(int types) { return in_size(types); }
ORACLE_API size_t oracle_out_size(int types) { return out_size(types); }
