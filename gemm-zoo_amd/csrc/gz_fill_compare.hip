// Harness kernels: seeded device fill and element-wise compare.
//
// Fill: element i is a pure function of (seed, i): Philox4x32-10 with counter
// {i_lo, i_hi, 0, 0} and key {seed_lo, seed_hi} -- the construction of
// test::populate_with_random (intel/test/utils.hpp:27-45: one philox4x32x10
// engine per element, keyed by seed and element id) and of the per-element
// curand states of nvidia/utils/fill_data.cuh:13-31.  The normal and uniform
// transforms use only IEEE-exact operations (+, *, /, sqrt, fma) in a fixed
// order, so a host implementation of the same expression tree reproduces the
// device values bit for bit.
//
// Compare: utils::compare_results (nvidia/utils/compare.cuh:14-47, absolute
// threshold) and test::compare_results (intel/test/utils.hpp:47-73, exact).
#include "gz_common.hpp"

namespace gz {

__device__ inline void philox4x32_10(uint32_t c0, uint32_t c1, uint32_t c2, uint32_t c3, uint32_t k0, uint32_t k1,
                                     uint32_t out[4]) {
#pragma unroll
  for (int r = 0; r < 10; r++) {
    const uint32_t hi0 = __umulhi(0xD2511F53u, c0), lo0 = 0xD2511F53u * c0;
    const uint32_t hi1 = __umulhi(0xCD9E8D57u, c2), lo1 = 0xCD9E8D57u * c2;
    const uint32_t n0 = hi1 ^ c1 ^ k0, n2 = hi0 ^ c3 ^ k1;
    c0 = n0; c1 = lo1; c2 = n2; c3 = lo0;
    k0 += 0x9E3779B9u;
    k1 += 0xBB67AE85u;
  }
  out[0] = c0; out[1] = c1; out[2] = c2; out[3] = c3;
}

__device__ inline float fma_rn(float a, float b, float c) { return __builtin_fmaf(a, b, c); }
// plain IEEE operations (contraction is off; fp32 divide and square root are correctly rounded by default)
__device__ inline float sub_rn(float a, float b) { return a - b; }
__device__ inline float div_rn(float a, float b) { return a / b; }
__device__ inline float sqrt_rn(float a) { return __builtin_sqrtf(a); }

// natural log on (0, 1]: exponent split + atanh series, IEEE-exact primitives only
__device__ inline float det_logf(float x) {
  const uint32_t u = __builtin_bit_cast(uint32_t, x);
  int e = (int)(u >> 23) - 127;
  float m = __builtin_bit_cast(float, (u & 0x007fffffu) | 0x3f800000u);
  if (m > 1.41421356f) { m = mul_rn(m, 0.5f); e += 1; }
  const float s = div_rn(sub_rn(m, 1.0f), add_rn(m, 1.0f));
  const float s2 = mul_rn(s, s);
  float p = 0.0909090909f;
  p = fma_rn(p, s2, 0.1111111111f);
  p = fma_rn(p, s2, 0.1428571429f);
  p = fma_rn(p, s2, 0.2f);
  p = fma_rn(p, s2, 0.3333333333f);
  p = fma_rn(p, s2, 1.0f);
  const float lm = mul_rn(add_rn(s, s), p);
  return fma_rn((float)e, 0.693147180559945f, lm);
}

// cos(2 pi u), u in [0,1): octant reduction is exact, then a Taylor polynomial on [0, pi/4]
__device__ inline float det_cos2pi(float u) {
  const float t = mul_rn(u, 8.0f);
  const int oct = (int)t;
  float r = sub_rn(t, (float)oct);
  if (oct & 1) r = sub_rn(1.0f, r);
  const float x = mul_rn(r, 0.785398163397448f);
  const float x2 = mul_rn(x, x);
  float sp = 2.7557319224e-6f;
  sp = fma_rn(sp, x2, -1.9841269841e-4f);
  sp = fma_rn(sp, x2, 8.3333333333e-3f);
  sp = fma_rn(sp, x2, -1.6666666667e-1f);
  sp = fma_rn(sp, x2, 1.0f);
  const float s = mul_rn(x, sp);
  float cp = 2.4801587302e-5f;
  cp = fma_rn(cp, x2, -1.3888888889e-3f);
  cp = fma_rn(cp, x2, 4.1666666667e-2f);
  cp = fma_rn(cp, x2, -0.5f);
  cp = fma_rn(cp, x2, 1.0f);
  const float c = cp;
  const bool swap = (((oct + 1) >> 1) & 1) != 0;   // octants 1,2,5,6 use the sine polynomial
  const float mag = swap ? s : c;
  const bool neg = oct >= 2 && oct <= 5;
  return neg ? -mag : mag;
}

__device__ inline float uniform01(uint32_t w) { return mul_rn((float)(w >> 8), 5.9604644775390625e-8f); }
__device__ inline float uniform01_open(uint32_t w) {
  return mul_rn((float)((w >> 8) + 1u), 5.9604644775390625e-8f);
}

__device__ inline float fill_value(int kind, float scale, uint64_t seed, uint64_t idx) {
  uint32_t w[4];
  philox4x32_10((uint32_t)idx, (uint32_t)(idx >> 32), 0u, 0u, (uint32_t)seed, (uint32_t)(seed >> 32), w);
  switch (kind) {
    case 0: return (float)(int8_t)(w[0] & 0xffu);
    case 1: {
      const float rad = sqrt_rn(mul_rn(-2.0f, det_logf(uniform01_open(w[0]))));
      return mul_rn(mul_rn(rad, det_cos2pi(uniform01(w[1]))), scale);
    }
    case 2: return mul_rn(fma_rn(uniform01(w[0]), 2.0f, -1.0f), scale);
    default: return (float)(int32_t)fma_rn(uniform01(w[0]), 4.0f, -2.0f);
  }
}

__global__ void __launch_bounds__(256) fill_kernel(void* dst, int64_t count, int dtype, int kind, float scale,
                                                   uint64_t seed) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (; i < count; i += stride) {
    const float v = fill_value(kind, scale, seed, (uint64_t)i);
    switch (dtype) {
      case 0: static_cast<int8_t*>(dst)[i] = (int8_t)v; break;
      case 1: static_cast<uint16_t*>(dst)[i] = f32_to_bf16(v); break;
      case 2: static_cast<uint16_t*>(dst)[i] = f32_to_f16(v); break;
      case 3: static_cast<float*>(dst)[i] = v; break;
      case 5: static_cast<uint8_t*>(dst)[i] = f32_to_e4m3(v); break;
      case 6: static_cast<uint8_t*>(dst)[i] = f32_to_e5m2(v); break;
      default: static_cast<int32_t*>(dst)[i] = (int32_t)v; break;
    }
  }
}

__device__ inline float load_as_float(const void* p, int64_t i, int dtype) {
  switch (dtype) {
    case 0: return (float)static_cast<const int8_t*>(p)[i];
    case 1: return bf16_to_f32(static_cast<const uint16_t*>(p)[i]);
    case 2: return f16_to_f32(static_cast<const uint16_t*>(p)[i]);
    case 3: return static_cast<const float*>(p)[i];
    default: return 0.0f;
  }
}

__global__ void __launch_bounds__(256) compare_kernel(const void* out, const void* ref, int64_t count, int dtype,
                                                      float thr, float rel, unsigned long long* ndiff) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  unsigned long long local = 0;
  for (; i < count; i += stride) {
    bool diff;
    if (dtype == 4) {
      const int32_t a = static_cast<const int32_t*>(out)[i], b = static_cast<const int32_t*>(ref)[i];
      diff = (thr == 0.0f && rel == 0.0f) ? (a != b)
                                          : (fabs((double)a - (double)b) > (double)thr + (double)rel * fabs((double)b));
    } else {
      const float a = load_as_float(out, i, dtype), b = load_as_float(ref, i, dtype);
      diff = (thr == 0.0f && rel == 0.0f) ? (a != b) : !(fabsf(a - b) <= thr + rel * fabsf(b));
    }
    local += diff ? 1u : 0u;
  }
  if (local) atomicAdd(ndiff, local);
}

}  // namespace gz

using namespace gz;

extern "C" {

int gz_fill(void* dst, int64_t count, int dtype, int kind, float scale, uint64_t seed, gz_stream stream) {
  if (count < 0 || dtype < 0 || dtype > 6 || kind < 0 || kind > 3) {
    set_error("gz_fill: bad argument (count=%lld dtype=%d kind=%d)", (long long)count, dtype, kind);
    return GZ_ERR_BAD_ARG;
  }
  if (count == 0) return GZ_OK;
  if (!dst) { set_error("gz_fill: dst is NULL"); return GZ_ERR_BAD_ARG; }
  const int64_t blocks = (count + 255) / 256;
  const dim3 grid((unsigned)(blocks < 16384 ? blocks : 16384)), block(256);
  hipLaunchKernelGGL(fill_kernel, grid, block, 0, static_cast<hipStream_t>(stream), dst, count, dtype, kind, scale,
                     seed);
  GZ_HIP_TRY(hipGetLastError());
  return GZ_OK;
}

int gz_compare_rel(const void* out, const void* ref, int64_t count, int dtype, float abs_threshold,
                   float rel_threshold, int64_t* num_different, gz_stream stream) {
  if (count < 0 || dtype < 0 || dtype > 4 || !(abs_threshold >= 0.0f) || !(rel_threshold >= 0.0f)) {
    set_error("gz_compare: bad argument (count=%lld dtype=%d)", (long long)count, dtype);
    return GZ_ERR_BAD_ARG;
  }
  if (num_different) *num_different = 0;
  if (count == 0) return GZ_OK;
  if (!out || !ref) { set_error("gz_compare: NULL array"); return GZ_ERR_BAD_ARG; }
  hipStream_t s = static_cast<hipStream_t>(stream);
  unsigned long long* d_count = nullptr;
  GZ_HIP_TRY(hipMalloc(&d_count, sizeof(*d_count)));
  unsigned long long h_count = 0;
  int st = GZ_OK;
  do {
    if (hipError_t e = hipMemcpyAsync(d_count, &h_count, sizeof(h_count), hipMemcpyHostToDevice, s); e != hipSuccess) {
      st = hip_fail(e, "hipMemcpyAsync");
      break;
    }
    const int64_t blocks = (count + 255) / 256;
    const dim3 grid((unsigned)(blocks < 16384 ? blocks : 16384)), block(256);
    hipLaunchKernelGGL(compare_kernel, grid, block, 0, s, out, ref, count, dtype, abs_threshold, rel_threshold, d_count);
    if (hipError_t e = hipGetLastError(); e != hipSuccess) { st = hip_fail(e, "compare launch"); break; }
    if (hipError_t e = hipMemcpyAsync(&h_count, d_count, sizeof(h_count), hipMemcpyDeviceToHost, s); e != hipSuccess) {
      st = hip_fail(e, "hipMemcpyAsync");
      break;
    }
    if (hipError_t e = hipStreamSynchronize(s); e != hipSuccess) { st = hip_fail(e, "hipStreamSynchronize"); break; }
  } while (0);
  (void)hipFree(d_count);
  if (st != GZ_OK) return st;
  if (num_different) *num_different = (int64_t)h_count;
  if (h_count) {
    set_error("verification failed: %llu of %lld elements differ", h_count, (long long)count);
    return GZ_ERR_MISMATCH;
  }
  return GZ_OK;
}

int gz_compare(const void* out, const void* ref, int64_t count, int dtype, float abs_threshold,
               int64_t* num_different, gz_stream stream) {
  return gz_compare_rel(out, ref, count, dtype, abs_threshold, 0.0f, num_different, stream);
}

}  // extern "C"
