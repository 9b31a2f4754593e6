// Shared device/host definitions for the gfx950 GEMM ladder.
#pragma once

// Every translation unit of the library is built with -ffp-contract=off and repeats it here:
// a*b+c written as two operations must round twice, so that the epilogue and the seeded fill
// produce the same bits as a host evaluation of the same expression.  Fused multiply-adds are
// always spelled __builtin_fmaf.
#pragma clang fp contract(off)

#include <hip/hip_runtime.h>
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

template <int TYPES> struct GemmArgs {
  using T = Traits<TYPES>;
  const typename T::in_t* A;
  const typename T::in_t* B;
  const typename T::out_t* C;
  typename T::out_t* D;
  int M, N, K;
  int layoutA, layoutB;
  typename T::scalar_t alpha, beta;
};

// ---------------------------------------------------------------------------
// 16-bit float helpers (device + host)
// ---------------------------------------------------------------------------
__host__ __device__ inline float bf16_to_f32(uint16_t h) {
  return __builtin_bit_cast(float, (uint32_t)h << 16);
}
__host__ __device__ inline uint16_t f32_to_bf16(float f) {
  uint32_t u = __builtin_bit_cast(uint32_t, f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}
__host__ __device__ inline float f16_to_f32(uint16_t h) {
  return (float)__builtin_bit_cast(_Float16, h);
}
__host__ __device__ inline uint16_t f32_to_f16(float f) {
  return __builtin_bit_cast(uint16_t, (_Float16)f);  // round-to-nearest-even
}

template <int TYPES> __host__ __device__ inline typename Traits<TYPES>::acc_t widen_in(typename Traits<TYPES>::in_t v) {
  if constexpr (TYPES == GZ_S8S8S32) return (int32_t)v;
  else if constexpr (TYPES == GZ_F16F16F16) return f16_to_f32(v);
  else if constexpr (TYPES == GZ_F32F32F32) return v;
  else return bf16_to_f32(v);
}

template <int TYPES> __host__ __device__ inline float round_out(float v) {
  if constexpr (TYPES == GZ_BF16BF16BF16) return bf16_to_f32(f32_to_bf16(v));
  else if constexpr (TYPES == GZ_F16F16F16) return f16_to_f32(f32_to_f16(v));
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
  } else if constexpr (TYPES == GZ_BF16BF16BF16) {
    float v = round_out<TYPES>(acc);
    v = round_out<TYPES>(mul_rn(v, alpha));
    if (beta != 0.0f) {
      float bc = round_out<TYPES>(mul_rn(beta, bf16_to_f32(*c_ptr)));
      v = round_out<TYPES>(add_rn(v, bc));
    }
    return f32_to_bf16(v);
  } else {
    float v = round_out<TYPES>(acc);
    v = round_out<TYPES>(mul_rn(v, alpha));
    if (beta != 0.0f) {
      float bc = round_out<TYPES>(mul_rn(beta, f16_to_f32(*c_ptr)));
      v = round_out<TYPES>(add_rn(v, bc));
    }
    return f32_to_f16(v);
  }
}

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

// Launchers, one per rung, explicitly instantiated for the four type bundles in
// the rung's own translation unit.  Each returns a gz_status.
template <int TYPES> int launch_naive(const GemmArgs<TYPES>& g, int variant, hipStream_t s);
template <int TYPES> int launch_coalesced(const GemmArgs<TYPES>& g, int variant, hipStream_t s);
template <int TYPES> int launch_lds_tiled(const GemmArgs<TYPES>& g, int variant, hipStream_t s);
template <int TYPES> int launch_double_buffered(const GemmArgs<TYPES>& g, int variant, hipStream_t s);
template <int TYPES> int launch_mfma(const GemmArgs<TYPES>& g, int variant, hipStream_t s);
template <int TYPES> int launch_skinny(const GemmArgs<TYPES>& g, int variant, hipStream_t s);

}  // namespace gz
