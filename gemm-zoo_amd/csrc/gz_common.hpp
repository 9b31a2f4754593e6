// Shared device/host definitions for the gfx950 GEMM ladder.
#pragma once

// Every translation unit of the library is built with -ffp-contract=off and repeats it here:
// a*b+c written as two operations must round twice, so that the epilogue and the seeded fill
// produce the same bits as a host evaluation of the same expression.  Fused multiply-adds are
// always spelled __builtin_fmaf.
#pragma clang fp contract(off)

#include <hip/hip_runtime.h>
#include <atomic>
#include <stdint.h>

#include "../../include/gemm_zoo.h"

namespace gz {

// ---------------------------------------------------------------------------
// Type bundles.  `in_t` / `out_t` are storage types (16-bit floats are carried
// as raw bit patterns); `acc_t` is the accumulator; `scalar_t` carries alpha
// and beta, already rounded to the output type on the host.
// ---------------------------------------------------------------------------
template <int TYPES> struct Traits;

template <> struct Traits<GZ_S8S8S32> {
  using in_t = int8_t;
  using acc_t = int32_t;
  using out_t = int32_t;
  using scalar_t = int32_t;
  static constexpr bool is_int = true;
};
template <> struct Traits<GZ_BF16BF16F32> {
  using in_t = uint16_t;
  using acc_t = float;
  using out_t = float;
  using scalar_t = float;
  static constexpr bool is_int = false;
};
template <> struct Traits<GZ_BF16BF16BF16> {
  using in_t = uint16_t;
  using acc_t = float;
  using out_t = uint16_t;
  using scalar_t = float;
  static constexpr bool is_int = false;
};
template <> struct Traits<GZ_F16F16F16> {
  using in_t = uint16_t;
  using acc_t = float;
  using out_t = uint16_t;
  using scalar_t = float;
  static constexpr bool is_int = false;
};

template <> struct Traits<GZ_F32F32F32> {
  using in_t = float;
  using acc_t = float;
  using out_t = float;
  using scalar_t = float;
  static constexpr bool is_int = false;
};

template <> struct Traits<GZ_E4M3E4M3F16> {
  using in_t = uint8_t;
  using acc_t = float;
  using out_t = uint16_t;
  using scalar_t = float;
  static constexpr bool is_int = false;
};
template <> struct Traits<GZ_E5M2E5M2F16> {
  using in_t = uint8_t;
  using acc_t = float;
  using out_t = uint16_t;
  using scalar_t = float;
  static constexpr bool is_int = false;
};

// 16-bit running sums (the reference kernels' own accumulators, opt-in): bf16 in chunks of 16 k, fp16 in chunks of 8
template <> struct Traits<GZ_BF16BF16BF16_ACC16> : Traits<GZ_BF16BF16BF16> {};
template <> struct Traits<GZ_F16F16F16_ACC16> : Traits<GZ_F16F16F16> {};
constexpr bool is_acc16(int types) { return types == GZ_BF16BF16BF16_ACC16 || types == GZ_F16F16F16_ACC16; }
constexpr int acc16_chunk(int types) { return types == GZ_BF16BF16BF16_ACC16 ? 16 : types == GZ_F16F16F16_ACC16 ? 8 : 0; }

constexpr bool is_fp8(int types) { return types == GZ_E4M3E4M3F16 || types == GZ_E5M2E5M2F16; }
constexpr bool out_is_f16(int types) { return types == GZ_F16F16F16 || types == GZ_F16F16F16_ACC16 || is_fp8(types); }

template <int TYPES> struct GemmArgs {
  using T = Traits<TYPES>;
  const typename T::in_t* A;
  const typename T::in_t* B;
  const typename T::out_t* C;
  typename T::out_t* D;
  int M, N, K;
  int layoutA, layoutB;
  typename T::scalar_t alpha, beta;
  int store_hint;   // MFMA rung, set by the launcher: bit 0 = the stores of D carry the non-temporal hint, bit 1 = the loads of C
  // Leading dimensions in elements (nvidia/kernels/generic_gemm.cuh:6-8 takes the same four): the distance between
  // consecutive lines of an operand - rows of a row-major A (at least K) or columns of a column-major one (at least
  // M), K rows of a row-major B (at least N) or columns of a column-major one (at least K), rows of C and of D (at
  // least N).  The packed entry points set them to those minima; the MFMA launcher also uses them to run a range of
  // rows or columns of a problem as a launch of its own.  Every index is formed in 64 bits: a matrix may hold 2^31
  // elements and more, its extents and leading dimensions stay below 2^31.
  int64_t lda, ldb, ldc, ldd;
};

// ---------------------------------------------------------------------------
// 16-bit float helpers (device + host)
// ---------------------------------------------------------------------------
__host__ __device__ inline float bf16_to_f32(uint16_t h) {
  return __builtin_bit_cast(float, (uint32_t)h << 16);
}
// On the device the conversion is one instruction (v_cvt_pk_bf16_f32); run over all 2^32 bit patterns it gave what
// the arithmetic below gives, NaNs included.  In a kernel whose output is bf16 the arithmetic, three roundings per
// element, cost more than the stores (4096 x 4096 x 128: 36 us, 21 us with fp32 output).
__host__ __device__ inline uint16_t f32_to_bf16(float f) {
#if defined(__HIP_DEVICE_COMPILE__)
  return __builtin_bit_cast(uint16_t, (__bf16)f);
#endif
  const uint32_t u = __builtin_bit_cast(uint32_t, f);
  const uint32_t rounded = u + 0x7fffu + ((u >> 16) & 1u);   // round to nearest even
  const uint32_t quiet = u | 0x00400000u;                    // NaN: keep the sign and payload, set the quiet bit
  return (uint16_t)(((u & 0x7fffffffu) > 0x7f800000u ? quiet : rounded) >> 16);
}
__host__ __device__ inline float f16_to_f32(uint16_t h) {
  return (float)__builtin_bit_cast(_Float16, h);
}
__host__ __device__ inline uint16_t f32_to_f16(float f) {
  return __builtin_bit_cast(uint16_t, (_Float16)f);  // round-to-nearest-even
}

// ---------------------------------------------------------------------------
// OCP 8-bit floats (device + host).  e5m2 is the upper byte of an IEEE half.  e4m3 has bias 7, no infinities,
// one NaN code per sign (exponent and mantissa all ones) and subnormals m * 2^-9.
// ---------------------------------------------------------------------------
__host__ __device__ inline float e5m2_to_f32(uint8_t b) { return f16_to_f32((uint16_t)((uint16_t)b << 8)); }
__host__ __device__ inline float e4m3_to_f32(uint8_t b) {
  const uint32_t s = (uint32_t)(b & 0x80u) << 24, e = (b >> 3) & 15u, m = b & 7u;
  if (e == 15u && m == 7u) return __builtin_bit_cast(float, s | 0x7fc00000u);
  if (e == 0u) return __builtin_bit_cast(float, s | __builtin_bit_cast(uint32_t, (float)m * 0x1p-9f));
  return __builtin_bit_cast(float, s | ((e + 120u) << 23) | (m << 20));
}
// fp32 -> 8-bit float with EXP exponent and MAN mantissa bits: round to nearest even, values beyond the largest
// finite one saturate to it (also infinities), NaN gives the all-ones code.
template <int EXP, int MAN> __host__ __device__ inline uint8_t f32_to_fp8(float f) {
  constexpr int BIAS = (1 << (EXP - 1)) - 1;
  // largest finite: e4m3 keeps the top exponent for numbers (mantissa 110), e5m2 gives it to inf / NaN
  constexpr uint32_t MAX_CODE = EXP == 4 ? 0x7eu : 0x7bu;
  const uint32_t u = __builtin_bit_cast(uint32_t, f);
  const uint8_t sign = (uint8_t)((u >> 24) & 0x80u);
  const uint32_t a = u & 0x7fffffffu;
  if (a > 0x7f800000u) return (uint8_t)(sign | 0x7fu);
  int e = (int)(a >> 23) - 127;
  if (e < 1 - BIAS) e = 1 - BIAS;                   // subnormal range shares the smallest normal's spacing
  if (e > BIAS + 1) return (uint8_t)(sign | MAX_CODE);
  // spacing of the target format around |f| is 2^(e - MAN); scaling by a power of two is exact
  const float inv_ulp = __builtin_bit_cast(float, (uint32_t)(127 - (e - MAN)) << 23);
  const uint32_t q = (uint32_t)__builtin_rintf(__builtin_bit_cast(float, a) * inv_ulp);  // 0 .. 2^(MAN+1)
  // q counts spacings from zero of this binade's grid: code = ((e + BIAS - 1) << MAN) + q also carries a
  // rounding up into the next binade and the subnormal / normal boundary
  const uint32_t code = ((uint32_t)(e + BIAS - 1) << MAN) + q;
  return (uint8_t)(sign | (code > MAX_CODE ? MAX_CODE : code));
}
__host__ __device__ inline uint8_t f32_to_e4m3(float f) { return f32_to_fp8<4, 3>(f); }
__host__ __device__ inline uint8_t f32_to_e5m2(float f) { return f32_to_fp8<5, 2>(f); }

template <int TYPES> __host__ __device__ inline typename Traits<TYPES>::acc_t widen_in(typename Traits<TYPES>::in_t v) {
  if constexpr (TYPES == GZ_S8S8S32) return (int32_t)v;
  else if constexpr (TYPES == GZ_E4M3E4M3F16) return e4m3_to_f32(v);
  else if constexpr (TYPES == GZ_E5M2E5M2F16) return e5m2_to_f32(v);
  else if constexpr (TYPES == GZ_F16F16F16 || TYPES == GZ_F16F16F16_ACC16) return f16_to_f32(v);
  else if constexpr (TYPES == GZ_F32F32F32) return v;
  else return bf16_to_f32(v);
}

template <int TYPES> __host__ __device__ inline float round_out(float v) {
  if constexpr (TYPES == GZ_BF16BF16BF16 || TYPES == GZ_BF16BF16BF16_ACC16) return bf16_to_f32(f32_to_bf16(v));
  else if constexpr (out_is_f16(TYPES)) return f16_to_f32(f32_to_f16(v));
  else return v;
}

// Explicit single-rounding fp32 operations: the epilogue must not be fused into
// an FMA, so that its value is the same on every rung.
__device__ inline float mul_rn(float a, float b) { return a * b; }
__device__ inline float add_rn(float a, float b) { return a + b; }

// Epilogue shared by every rung.  `c_ptr` is dereferenced only when beta != 0.
template <int TYPES>
__device__ inline typename Traits<TYPES>::out_t epilogue(typename Traits<TYPES>::acc_t acc,
                                                         typename Traits<TYPES>::scalar_t alpha,
                                                         typename Traits<TYPES>::scalar_t beta,
                                                         const typename Traits<TYPES>::out_t* c_ptr) {
  if constexpr (TYPES == GZ_S8S8S32) {
    uint32_t v = (uint32_t)alpha * (uint32_t)acc;
    if (beta != 0) v += (uint32_t)beta * (uint32_t)(*c_ptr);
    return (int32_t)v;
  } else if constexpr (TYPES == GZ_BF16BF16F32 || TYPES == GZ_F32F32F32) {
    float v = mul_rn(acc, alpha);
    if (beta != 0.0f) v = add_rn(v, mul_rn(beta, *c_ptr));
    return v;
  } else if constexpr (TYPES == GZ_F16F16F16_ACC16) {
    // nvidia/kernels/sm_80/fp16_mma_gemm.cuh:279-290: mul.f16x2 beta * c, then fma.rn.f16x2 alpha * acc + that;
    // acc, alpha and beta hold fp16 values, so the conversions down are exact and v_fma_f16 rounds once
    _Float16 bc = (_Float16)0.0f;
    if (beta != 0.0f) {
      float q = mul_rn(beta, f16_to_f32(*c_ptr));
      asm("" : "+v"(q));
      bc = (_Float16)q;
    }
    const _Float16 d = __builtin_fmaf16((_Float16)alpha, (_Float16)acc, bc);
    return __builtin_bit_cast(uint16_t, d);
  } else if constexpr (TYPES == GZ_BF16BF16BF16 || TYPES == GZ_BF16BF16BF16_ACC16) {
    float v = round_out<TYPES>(acc);
    v = round_out<TYPES>(mul_rn(v, alpha));
    if (beta != 0.0f) {
      float bc = round_out<TYPES>(mul_rn(beta, bf16_to_f32(*c_ptr)));
      v = round_out<TYPES>(add_rn(v, bc));
    }
    return f32_to_bf16(v);
  } else {
    // The products pass through an empty asm statement before they are rounded to fp16: otherwise the compiler
    // merges multiply and conversion into v_fma_mixlo_f16 with a +0 addend, which turns a product of -0 into +0.
    float v = round_out<TYPES>(acc);
    float p = mul_rn(v, alpha);
    asm("" : "+v"(p));
    v = round_out<TYPES>(p);
    if (beta != 0.0f) {
      float q = mul_rn(beta, f16_to_f32(*c_ptr));
      asm("" : "+v"(q));
      const float bc = round_out<TYPES>(q);
      v = round_out<TYPES>(add_rn(v, bc));
    }
    return f32_to_f16(v);
  }
}

// 16-bit running sums on the scalar rungs: `part` collects the exact products of one chunk in fp32, in k order; at the
// chunk's last k it is folded into `acc`, which holds a value of the output type.  k and k_end (the first k that
// does not exist) count from the same origin, a multiple of the chunk; elements past k_end that a kernel zero-fills
// add exact zeros, and a chunk made of such elements only is not folded (it would turn a running sum of -0 into +0).
// Types with an fp32 / int32 accumulator use `acc` alone.  finish() folds a last, shorter chunk.
template <int TYPES> struct RunningSum {
  using acc_t = typename Traits<TYPES>::acc_t;
  acc_t acc = 0, part = 0;
  __device__ inline void mac(acc_t a, acc_t b, int k, int k_end) {
    if constexpr (Traits<TYPES>::is_int) {
      acc += a * b;
    } else if constexpr (!is_acc16(TYPES)) {
      acc = __builtin_fmaf(a, b, acc);  // a*b is exact in fp32 for 8- and 16-bit inputs; fp32 inputs: fused by definition
    } else {
      part = __builtin_fmaf(a, b, part);
      if ((k & (acc16_chunk(TYPES) - 1)) == acc16_chunk(TYPES) - 1 && k - (acc16_chunk(TYPES) - 1) < k_end) fold();
    }
  }
  __device__ inline void fold() {
    if constexpr (is_acc16(TYPES)) {
      acc = round_out<TYPES>(add_rn(acc, part));
      part = 0;
    }
  }
  __device__ inline acc_t finish(int k_done) {   // k_done: one past the last k handed to mac()
    if constexpr (is_acc16(TYPES)) {
      if (k_done & (acc16_chunk(TYPES) - 1)) fold();
    }
    return acc;
  }
};

// Same epilogue on an already-loaded C value (for vectorised C loads).
template <int TYPES>
__device__ inline typename Traits<TYPES>::out_t epilogue_v(typename Traits<TYPES>::acc_t acc,
                                                           typename Traits<TYPES>::scalar_t alpha,
                                                           typename Traits<TYPES>::scalar_t beta,
                                                           typename Traits<TYPES>::out_t c_val) {
  return epilogue<TYPES>(acc, alpha, beta, &c_val);
}

// ---------------------------------------------------------------------------
// Status plumbing shared by the launchers
// ---------------------------------------------------------------------------
void set_error(const char* fmt, ...);
int hip_fail(hipError_t e, const char* what);

#define GZ_HIP_TRY(expr)                                      \
  do {                                                        \
    hipError_t _e = (expr);                                   \
    if (_e != hipSuccess) return ::gz::hip_fail(_e, #expr);   \
  } while (0)

inline int ceil_div(int a, int b) { return (a + b - 1) / b; }

// Compute units of the device that is current on the calling thread (queried once per device, then cached; 256
// if the query fails), and that device's index: what the launchers size their grids and splits for, so that
// gz_plan(num_cus = 0) and the launch agree on any part.
int device_compute_units();
int current_device_index();

// Device memory beyond the caller's matrices for a launch on stream `s` (partial sums of the stream-K launches): at
// least `bytes`, 256-byte aligned, valid until the next call for the same stream.  From the library's own pool
// (one buffer per device and stream, grown with hipMalloc when a call needs more), or - inside the entry point that
// allocates nothing - the static buffer, which refuses what it cannot hold.  Returns a gz_status.
int workspace_acquire(size_t bytes, hipStream_t s, void** out);
// The most workspace_acquire can give on the calling thread right now: unbounded from the pool, the size of the static
// buffer inside the entry point that allocates nothing.  The launcher's own choice stays within it.
size_t workspace_limit();

// Raises a kernel's dynamic LDS limit once per device instead of on every launch.
#define GZ_SET_LDS_LIMIT(kern, bytes)                                                                        \
  do {                                                                                                        \
    static std::atomic<uint64_t> gz_lds_set_{0};                                                              \
    const uint64_t gz_bit_ = 1ull << (::gz::current_device_index() & 63);                                     \
    if (!(gz_lds_set_.load(std::memory_order_acquire) & gz_bit_)) {                                           \
      GZ_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(kern),                                     \
                                     hipFuncAttributeMaxDynamicSharedMemorySize, (int)(bytes)));              \
      gz_lds_set_.fetch_or(gz_bit_, std::memory_order_release);                                               \
    }                                                                                                         \
  } while (0)

// Launchers, one per rung, explicitly instantiated for every type bundle in
// the rung's own translation unit.  Each returns a gz_status.
template <int TYPES> int launch_naive(const GemmArgs<TYPES>& g, int variant, hipStream_t s);
template <int TYPES> int launch_coalesced(const GemmArgs<TYPES>& g, int variant, hipStream_t s);
template <int TYPES> int launch_lds_tiled(const GemmArgs<TYPES>& g, int variant, hipStream_t s);
template <int TYPES> int launch_double_buffered(const GemmArgs<TYPES>& g, int variant, hipStream_t s);
template <int TYPES> int launch_mfma(const GemmArgs<TYPES>& g, int variant, hipStream_t s);
template <int TYPES> int launch_skinny(const GemmArgs<TYPES>& g, int variant, hipStream_t s);

}  // namespace gz
