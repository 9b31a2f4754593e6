// gemm-zoo's kernel-functor surface on top of the C ABI (gemm_zoo.h).
//
// Concept kept from the reference (nvidia/kernel_functors/*.cuh, intel/xe_gemm_*.hpp):
//     Kernel(std::size_t m, std::size_t n, std::size_t k, const hipDeviceProp_t&);
//     void operator()(const TIn* a, const TIn* b, const TOut* c, TOut* d, TOut alpha, TOut beta, hipStream_t);
// so that benchmark::benchmark<Kernel, TIn, TOut>(sizes, alpha, beta) drivers compile as they are, with
// cudaDeviceProp -> hipDeviceProp_t and cudaStream_t -> hipStream_t.  The constructor resolves the launch
// plan (the reference's grid / block / shared-memory computation) and rejects what the rung cannot run;
// operator() is asynchronous on the caller's stream.  Differences, all additive:
//   * A and B carry a layout (trailing template parameters, row-major by default as in the reference);
//   * the leading tile integers of the tiled / MMA functors are accepted as written in the reference's
//     drivers (they were tuned for another machine) and are a hint: the launcher chooses the gfx950 tile
//     configuration from the problem, and shapes need not be tile multiples.  mfma_gemm_variant<> pins one;
//   * errors of operator() throw std::runtime_error instead of ending the process.
#pragma once

#include <hip/hip_runtime_api.h>

#include <cstddef>
#include <cstdint>
#include <stdexcept>
#include <string>
#include <type_traits>

#include "../gemm_zoo.h"
#include "../gemm_zoo_hipblaslt.h"

namespace gemm_zoo {

// 16-bit storage types (bit patterns); enough for hosts that only move data around.
struct bf16_t { uint16_t bits; };
struct half_t { uint16_t bits; };
// Output types that also ask for the reference kernels' own 16-bit running sum instead of fp32 accumulation
// (bf16: intel/kernels/xe_gemm_bf16_bf16_bf16_m8k16.hpp:88-107; fp16: nvidia/kernels/sm_80/fp16_mma_gemm.cuh:179,
// 279-290): same storage as bf16_t / half_t, e.g. fp16_mma_gemm<half_t, half_acc16_t>.
struct bf16_acc16_t { uint16_t bits; };
struct half_acc16_t { uint16_t bits; };
// OCP 8-bit floats (the formats of __nv_fp8_e4m3 / __nv_fp8_e5m2), inputs only
struct e4m3_t { uint8_t bits; };
struct e5m2_t { uint8_t bits; };

enum class layout : int { row_major = GZ_ROW_MAJOR, col_major = GZ_COL_MAJOR };

namespace detail {
inline float bits_to_float(uint32_t u) { float f; __builtin_memcpy(&f, &u, 4); return f; }
inline float to_float(float v) { return v; }
inline float to_float(int32_t v) { return (float)v; }
inline float to_float(bf16_t v) { return bits_to_float((uint32_t)v.bits << 16); }
inline float to_float(half_t v) {
  _Float16 h; __builtin_memcpy(&h, &v.bits, 2); return (float)h;
}
inline float to_float(bf16_acc16_t v) { return to_float(bf16_t{v.bits}); }
inline float to_float(half_acc16_t v) { return to_float(half_t{v.bits}); }

template <typename TIn, typename TOut> struct bundle;  // (TIn, TOut) -> gz_types
template <> struct bundle<int8_t, int32_t> { static constexpr int value = GZ_S8S8S32; };
template <> struct bundle<bf16_t, float> { static constexpr int value = GZ_BF16BF16F32; };
template <> struct bundle<bf16_t, bf16_t> { static constexpr int value = GZ_BF16BF16BF16; };
template <> struct bundle<half_t, half_t> { static constexpr int value = GZ_F16F16F16; };
template <> struct bundle<bf16_t, bf16_acc16_t> { static constexpr int value = GZ_BF16BF16BF16_ACC16; };
template <> struct bundle<half_t, half_acc16_t> { static constexpr int value = GZ_F16F16F16_ACC16; };
template <> struct bundle<float, float> { static constexpr int value = GZ_F32F32F32; };  // the reference's ladder drivers
// nvidia/bench/bench_cublaslt_e4m3.cu:9-11, bench_cublaslt_e5m2.cu:9-11
template <> struct bundle<e4m3_t, half_t> { static constexpr int value = GZ_E4M3E4M3F16; };
template <> struct bundle<e5m2_t, half_t> { static constexpr int value = GZ_E5M2E5M2F16; };

template <typename TIn, typename TOut, layout LA, layout LB> class functor_base {
 public:
  static constexpr int types = bundle<TIn, TOut>::value;
  const gz_plan_t& plan() const { return plan_; }

  void operator()(const TIn* a, const TIn* b, const TOut* c, TOut* d, const TOut alpha, const TOut beta,
                  hipStream_t stream) const {
    int st;
    if constexpr (types == GZ_S8S8S32) {
      st = gz_gemm_s8s8s32(a, b, c, d, (int64_t)m_, (int64_t)n_, (int64_t)k_, (int)LA, (int)LB, alpha, beta, rung_,
                           variant_, stream);
    } else {
      st = gz_gemm(types, a, b, c, d, (int64_t)m_, (int64_t)n_, (int64_t)k_, (int)LA, (int)LB, to_float(alpha),
                   to_float(beta), rung_, variant_, stream);
    }
    if (st != GZ_OK) throw std::runtime_error(std::string("gemm_zoo: ") + gz_last_error());
  }

 protected:
  functor_base(std::size_t m, std::size_t n, std::size_t k, int rung, int variant, int num_cus, int lds_per_cu)
      : m_(m), n_(n), k_(k), rung_(rung), variant_(variant) {
    const int st = gz_plan(types, (int64_t)m, (int64_t)n, (int64_t)k, (int)LA, (int)LB, rung, variant, num_cus,
                           lds_per_cu, &plan_);
    if (st != GZ_OK) throw std::runtime_error(std::string("gemm_zoo: ") + gz_last_error());
  }
  std::size_t m_, n_, k_;
  int rung_, variant_;
  gz_plan_t plan_;
};

inline int cus(const hipDeviceProp_t& p) { return p.multiProcessorCount; }
inline int lds(const hipDeviceProp_t& p) { return (int)p.maxSharedMemoryPerMultiProcessor; }

// tile integers of the reference drivers are a hint only (0: launcher's choice)
constexpr int mfma_variant_for(int /*M*/, int /*N*/) { return 0; }
}  // namespace detail

namespace kernel_functors {

#define GZ_FUNCTOR_COMMON(NAME, RUNG, VARIANT)                                                                   \
  using base = detail::functor_base<TIn, TOut, LA, LB>;                                                          \
  NAME(std::size_t m, std::size_t n, std::size_t k, const hipDeviceProp_t& properties)                            \
      : base(m, n, k, RUNG, VARIANT, detail::cus(properties), detail::lds(properties)) {}

// nvidia/kernel_functors/naive_gemm.cuh:12-31
template <typename TIn, typename TOut, layout LA = layout::row_major, layout LB = layout::row_major>
struct naive_gemm : detail::functor_base<TIn, TOut, LA, LB> {
  GZ_FUNCTOR_COMMON(naive_gemm, GZ_RUNG_NAIVE, 0)
};

// nvidia/kernel_functors/generic_gemm.cuh:14-41 -- the any-shape fallback; three-argument constructor as there
template <typename TIn, typename TOut, layout LA = layout::row_major, layout LB = layout::row_major>
struct generic_gemm : detail::functor_base<TIn, TOut, LA, LB> {
  generic_gemm(std::size_t m, std::size_t n, std::size_t k)
      : detail::functor_base<TIn, TOut, LA, LB>(m, n, k, GZ_RUNG_LDS_TILED, 0, 0, 0) {}
};

// gfx950 rung with no counterpart of its own in the reference: layout-aware lanes, 128-bit global loads
template <typename TIn, typename TOut, layout LA = layout::row_major, layout LB = layout::row_major>
struct coalesced_gemm : detail::functor_base<TIn, TOut, LA, LB> {
  GZ_FUNCTOR_COMMON(coalesced_gemm, GZ_RUNG_COALESCED, 0)
};

// nvidia/kernel_functors/smem_tiled_gemm.cuh:14-51 and rmem_tiled_gemm.cuh:15-55 (LDS tiles + register blocks)
template <typename TIn, typename TOut, int M = 64, int N = 64, int K = 32, layout LA = layout::row_major,
          layout LB = layout::row_major>
struct smem_tiled_gemm : detail::functor_base<TIn, TOut, LA, LB> {
  GZ_FUNCTOR_COMMON(smem_tiled_gemm, GZ_RUNG_LDS_TILED, 0)
};
template <typename TIn, typename TOut, int M = 64, int N = 64, int K = 32, int TM = 4, int TN = 4, int TK = 1,
          layout LA = layout::row_major, layout LB = layout::row_major>
struct rmem_tiled_gemm : detail::functor_base<TIn, TOut, LA, LB> {
  GZ_FUNCTOR_COMMON(rmem_tiled_gemm, GZ_RUNG_LDS_TILED, 0)
};

// nvidia/kernel_functors/double_buffered_gemm.cuh:15-57 and async_buffered_gemm.cuh:16-58
template <typename TIn, typename TOut, int M = 64, int N = 64, int K = 32, int TM = 4, int TN = 4, int TK = 1,
          layout LA = layout::row_major, layout LB = layout::row_major>
struct double_buffered_gemm : detail::functor_base<TIn, TOut, LA, LB> {
  GZ_FUNCTOR_COMMON(double_buffered_gemm, GZ_RUNG_DOUBLE_BUFFERED, 0)
};
template <typename TIn, typename TOut, int M = 64, int N = 64, int K = 32, int TM = 4, int TN = 4, int TK = 1,
          layout LA = layout::row_major, layout LB = layout::row_major>
struct async_buffered_gemm : detail::functor_base<TIn, TOut, LA, LB> {
  GZ_FUNCTOR_COMMON(async_buffered_gemm, GZ_RUNG_DOUBLE_BUFFERED, 0)
};

// nvidia/kernel_functors/bf16_mma_gemm.cuh:16-72 (bf16 x bf16 -> f32; here also -> bf16)
template <typename TIn, typename TOut, int M = 256, int N = 256, int K = 64, layout LA = layout::row_major,
          layout LB = layout::row_major>
struct bf16_mma_gemm : detail::functor_base<TIn, TOut, LA, LB> {
  static_assert(std::is_same_v<TIn, bf16_t>, "bf16 inputs");
  GZ_FUNCTOR_COMMON(bf16_mma_gemm, GZ_RUNG_MFMA, detail::mfma_variant_for(M, N))
};

// nvidia/kernel_functors/fp16_mma_gemm.cuh:16-70 (fp16 x fp16 -> fp16; fp32 accumulate with TOut = half_t, the
// reference's fp16 accumulate with TOut = half_acc16_t)
template <typename TIn, typename TOut, int M = 256, int N = 256, int K = 64, layout LA = layout::row_major,
          layout LB = layout::row_major>
struct fp16_mma_gemm : detail::functor_base<TIn, TOut, LA, LB> {
  static_assert(std::is_same_v<TIn, half_t> && (std::is_same_v<TOut, half_t> || std::is_same_v<TOut, half_acc16_t>),
                "fp16 in and out");
  GZ_FUNCTOR_COMMON(fp16_mma_gemm, GZ_RUNG_MFMA, detail::mfma_variant_for(M, N))
};

// nvidia/kernel_functors/tf32_mma_gemm.cuh:15-60 (fp32 x fp32 -> fp32 on the tensor cores).  gfx950 has no tf32 mode;
// the matrix-core path here is v_mfma_f32_32x32x2_f32, full fp32 products, so results are tighter than the reference's.
template <typename TIn, typename TOut, int M = 128, int N = 128, int K = 32, layout LA = layout::row_major,
          layout LB = layout::row_major>
struct tf32_mma_gemm : detail::functor_base<TIn, TOut, LA, LB> {
  static_assert(std::is_same_v<TIn, float> && std::is_same_v<TOut, float>, "fp32 in and out");
  GZ_FUNCTOR_COMMON(tf32_mma_gemm, GZ_RUNG_MFMA, detail::mfma_variant_for(M, N))
};
template <typename TIn, typename TOut, int M = 128, int N = 128, int K = 32, layout LA = layout::row_major,
          layout LB = layout::row_major>
using f32_mma_gemm = tf32_mma_gemm<TIn, TOut, M, N, K, LA, LB>;

// fp8 x fp8 -> fp16 on the matrix cores; no counterpart in the reference, which runs these types through cuBLASLt
// only (nvidia/bench/bench_cublaslt_e4m3.cu, bench_cublaslt_e5m2.cu)
template <typename TIn, typename TOut, int M = 256, int N = 256, int K = 128, layout LA = layout::row_major,
          layout LB = layout::row_major>
struct fp8_mma_gemm : detail::functor_base<TIn, TOut, LA, LB> {
  static_assert((std::is_same_v<TIn, e4m3_t> || std::is_same_v<TIn, e5m2_t>) && std::is_same_v<TOut, half_t>,
                "fp8 in, fp16 out");
  GZ_FUNCTOR_COMMON(fp8_mma_gemm, GZ_RUNG_MFMA, detail::mfma_variant_for(M, N))
};

// int8 x int8 -> int32 on the matrix cores
template <typename TIn, typename TOut, int M = 256, int N = 256, int K = 128, layout LA = layout::row_major,
          layout LB = layout::row_major>
struct s8_mma_gemm : detail::functor_base<TIn, TOut, LA, LB> {
  static_assert(std::is_same_v<TIn, int8_t> && std::is_same_v<TOut, int32_t>, "s8 in, s32 out");
  GZ_FUNCTOR_COMMON(s8_mma_gemm, GZ_RUNG_MFMA, detail::mfma_variant_for(M, N))
};

// one pinned tile configuration of the MFMA rung (1 .. gz_variant_count)
template <typename TIn, typename TOut, int VARIANT, layout LA = layout::row_major, layout LB = layout::row_major>
struct mfma_gemm_variant : detail::functor_base<TIn, TOut, LA, LB> {
  GZ_FUNCTOR_COMMON(mfma_gemm_variant, GZ_RUNG_MFMA, VARIANT)
};

// launcher's choice: MFMA, or the weight-streaming kernel for decode shapes
template <typename TIn, typename TOut, layout LA = layout::row_major, layout LB = layout::row_major>
struct auto_gemm : detail::functor_base<TIn, TOut, LA, LB> {
  GZ_FUNCTOR_COMMON(auto_gemm, GZ_RUNG_AUTO, 0)
};
template <typename TIn, typename TOut, layout LA = layout::row_major, layout LB = layout::col_major>
struct skinny_gemm : detail::functor_base<TIn, TOut, LA, LB> {
  GZ_FUNCTOR_COMMON(skinny_gemm, GZ_RUNG_SKINNY, 0)
};
#undef GZ_FUNCTOR_COMMON

// nvidia/kernel_functors/cublaslt_gemm.cuh:15-125, with the descriptors released in the destructor
template <typename TIn, typename TOut, layout LA = layout::row_major, layout LB = layout::row_major>
struct hipblasLt_gemm {
  static constexpr int types = detail::bundle<TIn, TOut>::value;
  hipblasLt_gemm(std::size_t m, std::size_t n, std::size_t k, const hipDeviceProp_t&) {
    if (gz_hipblaslt_create(types, (int64_t)m, (int64_t)n, (int64_t)k, (int)LA, (int)LB, &plan_) != GZ_OK)
      throw std::runtime_error(std::string("hipBLASLt: ") + gz_hipblaslt_last_error());
  }
  hipblasLt_gemm(const hipblasLt_gemm&) = delete;
  hipblasLt_gemm& operator=(const hipblasLt_gemm&) = delete;
  ~hipblasLt_gemm() { gz_hipblaslt_destroy(plan_); }
  void operator()(const TIn* a, const TIn* b, const TOut* c, TOut* d, const TOut alpha, const TOut beta,
                  hipStream_t stream) const {
    if (gz_hipblaslt_run(plan_, a, b, c, d, detail::to_float(alpha), detail::to_float(beta), stream) != GZ_OK)
      throw std::runtime_error(std::string("hipBLASLt: ") + gz_hipblaslt_last_error());
  }

 private:
  void* plan_ = nullptr;
};
template <typename TIn, typename TOut, layout LA = layout::row_major, layout LB = layout::row_major>
using cublasLt_gemm = hipblasLt_gemm<TIn, TOut, LA, LB>;

}  // namespace kernel_functors

// The reference's typed entry points (intel/xe_gemm_*_m8k16.hpp:12-47) under their own names.
namespace intel {
template <typename TIn, typename TOut, layout LA = layout::row_major, layout LB = layout::row_major>
using gemm_s8_s8_s32_m8k16 = kernel_functors::auto_gemm<TIn, TOut, LA, LB>;
template <typename TIn, typename TOut, layout LA = layout::row_major, layout LB = layout::row_major>
using gemm_bf16_bf16_f32_m8k16 = kernel_functors::auto_gemm<TIn, TOut, LA, LB>;
template <typename TIn, typename TOut, layout LA = layout::row_major, layout LB = layout::row_major>
using gemm_bf16_bf16_bf16_m8k16 = kernel_functors::auto_gemm<TIn, TOut, LA, LB>;
}  // namespace intel

}  // namespace gemm_zoo

// Drivers written against the reference spell these namespaces.
namespace nvidia { namespace kernel_functors { using namespace ::gemm_zoo::kernel_functors; } }
namespace intel { using namespace ::gemm_zoo::intel; }
