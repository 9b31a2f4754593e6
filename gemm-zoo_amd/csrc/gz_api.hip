// extern "C" layer: argument checks, rung dispatch, launch planning, error text.
#include <stdarg.h>
#include <stdio.h>
#include <string.h>

#include <atomic>
#include <cmath>
#include <map>
#include <mutex>
#include <utility>

#include "gz_common.hpp"
#include "gz_mfma_cfg.hpp"
#include "gz_skinny_cfg.hpp"

// Scratch memory of gz_gemm_static_scratch: part of the device image, one copy per GPU.  In host code this name is
// a stand-in, not a device address: scratch_address() asks the runtime for the address once per device and
// everything else uses that pointer.
static __device__ __align__(256) unsigned char scratch[GZ_STATIC_SCRATCH_BYTES];

namespace gz {

static thread_local char g_err[512] = "";

void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
}

int hip_fail(hipError_t e, const char* what) {
  set_error("HIP error %d (%s) in %s", (int)e, hipGetErrorString(e), what);
  return GZ_ERR_HIP;
}

// ---------------------------------------------------------------------------
// Workspace of the stream-K launches
// ---------------------------------------------------------------------------
static thread_local bool t_static_scratch = false;   // set for the duration of a gz_gemm_static_scratch call

// Address of `scratch` on the device that is current: each GPU holds its own copy of the array at its own address.
static int scratch_address(void** out) {
  constexpr int MAX_DEVICES = 64;
  static std::atomic<void*> cached[MAX_DEVICES];
  const int dev = current_device_index();
  if (dev < 0 || dev >= MAX_DEVICES) { set_error("device index %d out of range", dev); return GZ_ERR_UNSUPPORTED; }
  void* p = cached[dev].load(std::memory_order_acquire);
  if (!p) {
    GZ_HIP_TRY(hipGetSymbolAddress((void**)&p, HIP_SYMBOL(scratch)));
    if (!p) { set_error("hipGetSymbolAddress returned no address for the static scratch buffer"); return GZ_ERR_HIP; }
    cached[dev].store(p, std::memory_order_release);
  }
  *out = p;
  return GZ_OK;
}

namespace {
struct PoolBuffer { void* ptr = nullptr; size_t bytes = 0; };
std::mutex g_pool_mutex;
std::map<std::pair<int, hipStream_t>, PoolBuffer> g_pool;   // never freed before the process ends
}  // namespace

size_t workspace_limit() { return t_static_scratch ? (size_t)GZ_STATIC_SCRATCH_BYTES : ~(size_t)0; }

int workspace_acquire(size_t bytes, hipStream_t s, void** out) {
  if (t_static_scratch) {   // no allocation on this path
    if (bytes > (size_t)GZ_STATIC_SCRATCH_BYTES) {
      set_error("this launch needs %zu bytes of scratch memory, the static buffer holds %lld: use gz_gemm, which "
                "allocates what it needs, or a variant without stream-K (5, 6)", bytes,
                (long long)GZ_STATIC_SCRATCH_BYTES);
      return GZ_ERR_UNSUPPORTED;
    }
    return scratch_address(out);
  }
  std::lock_guard<std::mutex> lock(g_pool_mutex);
  PoolBuffer& b = g_pool[{current_device_index(), s}];
  if (b.bytes < bytes) {
    if (b.ptr) {
      // work queued on this stream may still use the old buffer
      GZ_HIP_TRY(hipStreamSynchronize(s));
      GZ_HIP_TRY(hipFree(b.ptr));
      b.ptr = nullptr;
      b.bytes = 0;
    }
    const size_t want = (bytes + (size_t)(1 << 20) - 1) & ~((size_t)(1 << 20) - 1);
    GZ_HIP_TRY(hipMalloc(&b.ptr, want));
    b.bytes = want;
  }
  *out = b.ptr;
  return GZ_OK;
}

int current_device_index() {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) dev = 0;
  return dev;
}

int device_compute_units() {
  constexpr int MAX_DEVICES = 64;
  static std::atomic<int> cached[MAX_DEVICES];   // 0: not asked yet
  const int dev = current_device_index();
  if (dev < 0 || dev >= MAX_DEVICES) return 256;
  int cus = cached[dev].load(std::memory_order_relaxed);
  if (cus == 0) {
    int v = 0;
    if (hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || v <= 0) v = 256;
    cached[dev].store(v, std::memory_order_relaxed);
    cus = v;
  }
  return cus;
}

static const char* kRungNames[GZ_NUM_RUNGS] = {"naive", "coalesced", "lds_tiled", "double_buffered", "mfma", "skinny"};
static const char* kTypesNames[GZ_NUM_TYPES] = {"s8s8s32",   "bf16bf16f32", "bf16bf16bf16", "f16f16f16",
                                                "f32f32f32", "e4m3e4m3f16", "e5m2e5m2f16",
                                                "bf16bf16bf16_acc16", "f16f16f16_acc16"};

static int in_size(int types) { return (types == GZ_S8S8S32 || is_fp8(types)) ? 1 : types == GZ_F32F32F32 ? 4 : 2; }
static int out_size(int types) {
  return (types == GZ_S8S8S32 || types == GZ_BF16BF16F32 || types == GZ_F32F32F32) ? 4 : 2;
}

// Shape / enum checks common to gz_plan and the GEMM entry points.
static int check_problem(int types, int64_t M, int64_t N, int64_t K, int layoutA, int layoutB, int rung) {
  if (types < 0 || types >= GZ_NUM_TYPES) {
    set_error("unknown type bundle %d", types);
    return GZ_ERR_BAD_ARG;
  }
  if (M < 0 || N < 0 || K < 0) {
    set_error("negative size M=%lld N=%lld K=%lld", (long long)M, (long long)N, (long long)K);
    return GZ_ERR_BAD_ARG;
  }
  if ((layoutA != GZ_ROW_MAJOR && layoutA != GZ_COL_MAJOR) || (layoutB != GZ_ROW_MAJOR && layoutB != GZ_COL_MAJOR)) {
    set_error("unknown layout A=%d B=%d", layoutA, layoutB);
    return GZ_ERR_BAD_ARG;
  }
  if (rung < GZ_RUNG_AUTO || rung >= GZ_NUM_RUNGS) {
    set_error("unknown rung %d", rung);
    return GZ_ERR_BAD_ARG;
  }
  // extents and leading dimensions are 32-bit in the kernels; every index they form from them is 64-bit, so a matrix
  // may hold 2^31 elements and more
  const int64_t lim = (int64_t)1 << 31;
  if (M >= lim || N >= lim || K >= lim) {
    set_error("an extent of 2^31 or more is not supported (M=%lld N=%lld K=%lld)", (long long)M, (long long)N,
              (long long)K);
    return GZ_ERR_UNSUPPORTED;
  }
  return GZ_OK;
}

static int resolve_rung(int types, int64_t M, int64_t N, int64_t K, int layoutA, int layoutB, int rung) {
  if (rung != GZ_RUNG_AUTO) return rung;
  if (skinny_preferred(types, (int)M, (int)N, (int)K, layoutA, layoutB, 0)) return GZ_RUNG_SKINNY;
  return GZ_RUNG_MFMA;
}

// Leading dimensions: 0 stands for the packed value; otherwise at least the line's extent and below 2^31.
static int resolve_ld(const char* name, int64_t given, int64_t extent, int64_t* out) {
  if (given == 0) given = extent > 0 ? extent : 1;
  if (given < extent || given < 1) {
    set_error("%s = %lld is smaller than the %lld elements of a line", name, (long long)given, (long long)extent);
    return GZ_ERR_BAD_ARG;
  }
  if (given >= ((int64_t)1 << 31)) {
    set_error("%s = %lld: a leading dimension of 2^31 or more is not supported", name, (long long)given);
    return GZ_ERR_UNSUPPORTED;
  }
  *out = given;
  return GZ_OK;
}

struct LeadingDims { int64_t a, b, c, d; };   // 0: packed

template <int TYPES>
static int run(const void* A, const void* B, const void* C, void* D, int64_t M, int64_t N, int64_t K, int layoutA,
               int layoutB, typename Traits<TYPES>::scalar_t alpha, typename Traits<TYPES>::scalar_t beta, int rung,
               int variant, gz_stream stream, LeadingDims ld = LeadingDims{0, 0, 0, 0}) {
  using T = Traits<TYPES>;
  int st = check_problem(TYPES, M, N, K, layoutA, layoutB, rung);
  if (st != GZ_OK) return st;
  int64_t lda = 0, ldb = 0, ldc = 0, ldd = 0;
  if ((st = resolve_ld("lda", ld.a, layoutA == GZ_ROW_MAJOR ? K : M, &lda)) != GZ_OK) return st;
  if ((st = resolve_ld("ldb", ld.b, layoutB == GZ_ROW_MAJOR ? N : K, &ldb)) != GZ_OK) return st;
  if ((st = resolve_ld("ldc", ld.c, N, &ldc)) != GZ_OK) return st;
  if ((st = resolve_ld("ldd", ld.d, N, &ldd)) != GZ_OK) return st;
  if (M == 0 || N == 0) return GZ_OK;  // nothing to write
  if (!A && K > 0 && M > 0) { set_error("A is NULL"); return GZ_ERR_BAD_ARG; }
  if (!B && K > 0 && N > 0) { set_error("B is NULL"); return GZ_ERR_BAD_ARG; }
  if (!D) { set_error("D is NULL"); return GZ_ERR_BAD_ARG; }
  if (!C && beta != 0) { set_error("C is NULL but beta != 0"); return GZ_ERR_BAD_ARG; }
  if (variant < 0) { set_error("negative variant %d", variant); return GZ_ERR_BAD_ARG; }

  GemmArgs<TYPES> g;
  g.A = static_cast<const typename T::in_t*>(A);
  g.B = static_cast<const typename T::in_t*>(B);
  g.C = static_cast<const typename T::out_t*>(C);
  g.D = static_cast<typename T::out_t*>(D);
  g.M = (int)M; g.N = (int)N; g.K = (int)K;
  g.layoutA = layoutA; g.layoutB = layoutB;
  g.alpha = alpha; g.beta = beta;
  g.store_hint = 0;
  g.lda = lda; g.ldb = ldb; g.ldc = ldc; g.ldd = ldd;
  hipStream_t s = static_cast<hipStream_t>(stream);

  int resolved = resolve_rung(TYPES, M, N, K, layoutA, layoutB, rung);
  // the streaming kernel needs 16-byte aligned operands and lines; AUTO falls back to the tiled kernel otherwise
  if (rung == GZ_RUNG_AUTO && resolved == GZ_RUNG_SKINNY &&
      (((reinterpret_cast<uintptr_t>(A) | reinterpret_cast<uintptr_t>(B)) & 15u) || !skinny_lines_ok(lda, ldb)))
    resolved = GZ_RUNG_MFMA;
  switch (resolved) {
    case GZ_RUNG_NAIVE: return launch_naive<TYPES>(g, variant, s);
    case GZ_RUNG_COALESCED: return launch_coalesced<TYPES>(g, variant, s);
    case GZ_RUNG_LDS_TILED: return launch_lds_tiled<TYPES>(g, variant, s);
    case GZ_RUNG_DOUBLE_BUFFERED: return launch_double_buffered<TYPES>(g, variant, s);
    case GZ_RUNG_MFMA: return launch_mfma<TYPES>(g, variant, s);
    case GZ_RUNG_SKINNY: return launch_skinny<TYPES>(g, variant, s);
    default: break;
  }
  set_error("unknown rung %d", rung);
  return GZ_ERR_BAD_ARG;
}

}  // namespace gz

using namespace gz;

extern "C" {

int gz_gemm_s8s8s32(const int8_t* A, const int8_t* B, const int32_t* C, int32_t* D, int64_t M, int64_t N, int64_t K,
                    int layoutA, int layoutB, int32_t alpha, int32_t beta, int rung, int variant, gz_stream stream) {
  return run<GZ_S8S8S32>(A, B, C, D, M, N, K, layoutA, layoutB, alpha, beta, rung, variant, stream);
}

int gz_gemm_bf16bf16f32(const uint16_t* A, const uint16_t* B, const float* C, float* D, int64_t M, int64_t N,
                        int64_t K, int layoutA, int layoutB, float alpha, float beta, int rung, int variant,
                        gz_stream stream) {
  return run<GZ_BF16BF16F32>(A, B, C, D, M, N, K, layoutA, layoutB, alpha, beta, rung, variant, stream);
}

int gz_gemm_bf16bf16bf16(const uint16_t* A, const uint16_t* B, const uint16_t* C, uint16_t* D, int64_t M, int64_t N,
                         int64_t K, int layoutA, int layoutB, float alpha, float beta, int rung, int variant,
                         gz_stream stream) {
  return run<GZ_BF16BF16BF16>(A, B, C, D, M, N, K, layoutA, layoutB, round_out<GZ_BF16BF16BF16>(alpha),
                              round_out<GZ_BF16BF16BF16>(beta), rung, variant, stream);
}

int gz_gemm_f16f16f16(const uint16_t* A, const uint16_t* B, const uint16_t* C, uint16_t* D, int64_t M, int64_t N,
                      int64_t K, int layoutA, int layoutB, float alpha, float beta, int rung, int variant,
                      gz_stream stream) {
  return run<GZ_F16F16F16>(A, B, C, D, M, N, K, layoutA, layoutB, round_out<GZ_F16F16F16>(alpha),
                           round_out<GZ_F16F16F16>(beta), rung, variant, stream);
}

int gz_gemm_f32f32f32(const float* A, const float* B, const float* C, float* D, int64_t M, int64_t N, int64_t K,
                      int layoutA, int layoutB, float alpha, float beta, int rung, int variant, gz_stream stream) {
  return run<GZ_F32F32F32>(A, B, C, D, M, N, K, layoutA, layoutB, alpha, beta, rung, variant, stream);
}

int gz_gemm_e4m3e4m3f16(const uint8_t* A, const uint8_t* B, const uint16_t* C, uint16_t* D, int64_t M, int64_t N,
                        int64_t K, int layoutA, int layoutB, float alpha, float beta, int rung, int variant,
                        gz_stream stream) {
  return run<GZ_E4M3E4M3F16>(A, B, C, D, M, N, K, layoutA, layoutB, round_out<GZ_E4M3E4M3F16>(alpha),
                             round_out<GZ_E4M3E4M3F16>(beta), rung, variant, stream);
}

int gz_gemm_e5m2e5m2f16(const uint8_t* A, const uint8_t* B, const uint16_t* C, uint16_t* D, int64_t M, int64_t N,
                        int64_t K, int layoutA, int layoutB, float alpha, float beta, int rung, int variant,
                        gz_stream stream) {
  return run<GZ_E5M2E5M2F16>(A, B, C, D, M, N, K, layoutA, layoutB, round_out<GZ_E5M2E5M2F16>(alpha),
                             round_out<GZ_E5M2E5M2F16>(beta), rung, variant, stream);
}

int gz_gemm_bf16bf16bf16_acc16(const uint16_t* A, const uint16_t* B, const uint16_t* C, uint16_t* D, int64_t M,
                               int64_t N, int64_t K, int layoutA, int layoutB, float alpha, float beta, int rung,
                               int variant, gz_stream stream) {
  return run<GZ_BF16BF16BF16_ACC16>(A, B, C, D, M, N, K, layoutA, layoutB, round_out<GZ_BF16BF16BF16_ACC16>(alpha),
                                    round_out<GZ_BF16BF16BF16_ACC16>(beta), rung, variant, stream);
}

int gz_gemm_f16f16f16_acc16(const uint16_t* A, const uint16_t* B, const uint16_t* C, uint16_t* D, int64_t M,
                            int64_t N, int64_t K, int layoutA, int layoutB, float alpha, float beta, int rung,
                            int variant, gz_stream stream) {
  return run<GZ_F16F16F16_ACC16>(A, B, C, D, M, N, K, layoutA, layoutB, round_out<GZ_F16F16F16_ACC16>(alpha),
                                 round_out<GZ_F16F16F16_ACC16>(beta), rung, variant, stream);
}

// the typed launch behind gz_gemm and gz_gemm_ld (alpha and beta as doubles, rounded to the output type here as the
// typed entry points do)
static int gemm_any(int types, const void* A, const void* B, const void* C, void* D, int64_t M, int64_t N, int64_t K,
                    int layoutA, int layoutB, double alpha, double beta, int rung, int variant, gz_stream stream,
                    LeadingDims ld) {
  const float af = (float)alpha, bf = (float)beta;
  switch (types) {
    case GZ_S8S8S32:
      if (alpha != std::floor(alpha) || beta != std::floor(beta) || std::fabs(alpha) > 2147483647.0 ||
          std::fabs(beta) > 2147483647.0) {
        set_error("s8s8s32 needs integral alpha/beta that fit int32");
        return GZ_ERR_BAD_ARG;
      }
      return run<GZ_S8S8S32>(A, B, C, D, M, N, K, layoutA, layoutB, (int32_t)alpha, (int32_t)beta, rung, variant, stream, ld);
    case GZ_BF16BF16F32: return run<GZ_BF16BF16F32>(A, B, C, D, M, N, K, layoutA, layoutB, af, bf, rung, variant, stream, ld);
    case GZ_F32F32F32: return run<GZ_F32F32F32>(A, B, C, D, M, N, K, layoutA, layoutB, af, bf, rung, variant, stream, ld);
#define GZ_ROUNDED(TY) \
    case TY: return run<TY>(A, B, C, D, M, N, K, layoutA, layoutB, round_out<TY>(af), round_out<TY>(bf), rung, variant, stream, ld);
    GZ_ROUNDED(GZ_BF16BF16BF16)
    GZ_ROUNDED(GZ_F16F16F16)
    GZ_ROUNDED(GZ_E4M3E4M3F16)
    GZ_ROUNDED(GZ_E5M2E5M2F16)
    GZ_ROUNDED(GZ_BF16BF16BF16_ACC16)
    GZ_ROUNDED(GZ_F16F16F16_ACC16)
#undef GZ_ROUNDED
    default: break;
  }
  set_error("unknown type bundle %d", types);
  return GZ_ERR_BAD_ARG;
}

int gz_gemm(int types, const void* A, const void* B, const void* C, void* D, int64_t M, int64_t N, int64_t K,
            int layoutA, int layoutB, double alpha, double beta, int rung, int variant, gz_stream stream) {
  return gemm_any(types, A, B, C, D, M, N, K, layoutA, layoutB, alpha, beta, rung, variant, stream,
                  LeadingDims{0, 0, 0, 0});
}

int gz_gemm_ld(int types, const void* A, int64_t lda, const void* B, int64_t ldb, const void* C, int64_t ldc, void* D,
               int64_t ldd, int64_t M, int64_t N, int64_t K, int layoutA, int layoutB, double alpha, double beta,
               int rung, int variant, gz_stream stream) {
  if (lda < 0 || ldb < 0 || ldc < 0 || ldd < 0) {
    set_error("negative leading dimension lda=%lld ldb=%lld ldc=%lld ldd=%lld", (long long)lda, (long long)ldb,
              (long long)ldc, (long long)ldd);
    return GZ_ERR_BAD_ARG;
  }
  return gemm_any(types, A, B, C, D, M, N, K, layoutA, layoutB, alpha, beta, rung, variant, stream,
                  LeadingDims{lda, ldb, ldc, ldd});
}

int gz_device_props(int32_t* num_cus, int32_t* lds_per_cu) {
  int dev = 0;
  GZ_HIP_TRY(hipGetDevice(&dev));
  int cus = 0, lds = 0;
  GZ_HIP_TRY(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
  GZ_HIP_TRY(hipDeviceGetAttribute(&lds, hipDeviceAttributeMaxSharedMemoryPerMultiprocessor, dev));
  if (num_cus) *num_cus = cus;
  if (lds_per_cu) *lds_per_cu = lds;
  return GZ_OK;
}

int gz_gemm_static_scratch(int types, const void* A, const void* B, const void* C, void* D, int64_t M, int64_t N,
                           int64_t K, int layoutA, int layoutB, double alpha, double beta, int rung, int variant,
                           gz_stream stream) {
  struct Scope {   // the launchers below ask workspace_acquire, which looks at this flag
    Scope() { t_static_scratch = true; }
    ~Scope() { t_static_scratch = false; }
  } scope;
  return gz_gemm(types, A, B, C, D, M, N, K, layoutA, layoutB, alpha, beta, rung, variant, stream);
}

int gz_variant_count(int types, int rung) {
  if (types < 0 || types >= GZ_NUM_TYPES) return 0;
  switch (rung) {
    case GZ_RUNG_NAIVE: case GZ_RUNG_COALESCED: case GZ_RUNG_LDS_TILED: case GZ_RUNG_DOUBLE_BUFFERED: return 1;
    case GZ_RUNG_MFMA: return is_acc16(types) ? 1 : kNumMfmaCfgs;
    case GZ_RUNG_SKINNY: return (types == GZ_S8S8S32 || types == GZ_F32F32F32 || is_fp8(types) || is_acc16(types)) ? 0 : 1;
    default: return 0;
  }
}

// ws_limit: the most device memory beyond the matrices that the launch may use (what workspace_limit() will say
// inside the entry point the plan is asked for)
static int plan_impl(int types, int64_t M, int64_t N, int64_t K, int layoutA, int layoutB, int rung, int variant,
                     int num_cus, int lds_per_cu, size_t ws_limit, gz_plan_t* plan) {
  if (!plan) { set_error("plan is NULL"); return GZ_ERR_BAD_ARG; }
  int st = check_problem(types, M, N, K, layoutA, layoutB, rung);
  if (st != GZ_OK) return st;
  if (variant < 0) { set_error("negative variant %d", variant); return GZ_ERR_BAD_ARG; }
  if (num_cus <= 0) num_cus = 256;
  if (lds_per_cu <= 0) lds_per_cu = 160 * 1024;
  memset(plan, 0, sizeof(*plan));
  const int r = resolve_rung(types, M, N, K, layoutA, layoutB, rung);
  plan->rung = r;
  plan->split_k = 1;
  const int es = in_size(types);
  const int m = (int)M, n = (int)N, k = (int)K;
  const bool a_kc = layoutA == GZ_ROW_MAJOR, b_kc = layoutB == GZ_COL_MAJOR;
  // widest naturally aligned vector each operand allows (packed lines, 16-byte aligned base assumed)
  auto vec_bytes = [&](int extent) {
    int bytes = extent * es, v = 16;
    while (v > es && bytes % v) v >>= 1;
    return v;
  };
  plan->vector_bytes_a = vec_bytes(a_kc ? k : m);
  plan->vector_bytes_b = vec_bytes(b_kc ? k : n);
  switch (r) {
    case GZ_RUNG_NAIVE:
      if (variant != 0) { set_error("naive rung has a single variant"); return GZ_ERR_UNSUPPORTED; }
      plan->tile_m = 32; plan->tile_n = 32; plan->tile_k = 1; plan->threads = 1024;
      plan->grid = (int64_t)ceil_div(m, 32) * ceil_div(n, 32);
      plan->vector_bytes_a = plan->vector_bytes_b = es;
      return GZ_OK;
    case GZ_RUNG_COALESCED:
      if (variant != 0) { set_error("coalesced rung has a single variant"); return GZ_ERR_UNSUPPORTED; }
      plan->tile_m = 16; plan->tile_n = 64; plan->tile_k = 16 / es; plan->threads = 256;
      plan->grid = (int64_t)ceil_div(m, 16) * ceil_div(n, 64);
      return GZ_OK;
    case GZ_RUNG_LDS_TILED:
    case GZ_RUNG_DOUBLE_BUFFERED: {
      if (variant != 0) { set_error("rung has a single variant"); return GZ_ERR_UNSUPPORTED; }
      const int stages = r == GZ_RUNG_DOUBLE_BUFFERED ? 2 : 1;
      plan->tile_m = 64; plan->tile_n = 64; plan->tile_k = 32; plan->threads = 256;
      plan->lds_bytes = stages * 2 * 32 * (64 + 4) * 4;
      plan->grid = (int64_t)ceil_div(m, 64) * ceil_div(n, 64);
      return GZ_OK;
    }
    case GZ_RUNG_MFMA: {
      if (is_acc16(types)) {   // one kernel: 128 x 128 tile, four waves of 64 x 64, slabs of 32 k (rung4_mfma_acc16.hip)
        if (variant > 1) { set_error("mfma rung has a single variant for the 16-bit running-sum modes"); return GZ_ERR_UNSUPPORTED; }
        plan->variant = 1;
        plan->tile_m = 128; plan->tile_n = 128; plan->tile_k = 32; plan->wave_m = 64; plan->wave_n = 64;
        plan->threads = 256; plan->lds_bytes = 256 * (64 + 16);
        plan->grid = (int64_t)ceil_div(m, 128) * ceil_div(n, 128);
        return GZ_OK;
      }
      MfmaSplit tsp;
      // (column-major A and B: a few columns past a multiple of 256 are cut off first, as launch_mfma does)
      MfmaColSplit ccs;
      const bool cc_cut = variant == 0 && k > 0 && layoutA == GZ_COL_MAJOR && layoutB == GZ_COL_MAJOR &&
                          mfma_resolve_colsplit(types, m, n, k, layoutA, layoutB, num_cus, &ccs);
      const int n_ring = cc_cut ? ccs.cols_main : n;   // columns that the transposed problem covers
      if (MfmaCfg ct; mfma_transposed_ring(types, m, n_ring, k, layoutA, layoutB, variant, num_cus, &ct, cc_cut ? nullptr : &tsp)) {
        if (cc_cut) tsp.rows_main = 0;
        // column-major A and B: the ring kernel on the transposed problem (as launch_mfma, aligned operands assumed);
        // the configuration's rows run along N there
        plan->variant = ct.id;
        plan->tile_m = ct.bn; plan->tile_n = ct.bm; plan->tile_k = MFMA_SLAB_BYTES / es;
        plan->wave_m = ct.bn / ct.waves_m; plan->wave_n = ct.bm / ct.waves_n;
        plan->threads = ct.waves_m * ct.waves_n * 64;
        plan->lds_bytes = mfma_lds_bytes(ct);
        const int n_first = tsp.rows_main > 0 ? tsp.rows_main : n_ring;   // columns of the first launch
        plan->grid = (int64_t)ceil_div(n_first, ct.bm) * ceil_div(m, ct.bn);
        const int cls_t = mfma_shape_class(ct, es, n_first, m, k, GZ_ROW_MAJOR, GZ_ROW_MAJOR);
        if (ct.ring == 1 && (cls_t == MFMA_SHAPE_WHOLE || (cls_t == MFMA_SHAPE_RAGGED_MN && ct.bm == 256)))
          plan->grid = mfma_persistent_grid(plan->grid, num_cus);
        if (tsp.rows_main > 0) {   // the remaining columns in a second launch
          plan->tail_cols = n - tsp.rows_main;
          plan->tail_tile_m = tsp.tail.bn;
          plan->tail_tile_n = tsp.tail.bm;
          plan->tail_grid = (int64_t)ceil_div(n - tsp.rows_main, tsp.tail.bm) * ceil_div(m, tsp.tail.bn);
        }
        if (cc_cut) {   // the cut-off columns: dot products, or tiles of the problem as given
          plan->tail_cols = n - ccs.cols_main;
          plan->tail_tile_m = ccs.strip ? 16 : ccs.tail.bm;
          plan->tail_tile_n = ccs.strip ? plan->tail_cols : ccs.tail.bn;
          plan->tail_grid = ccs.strip ? ceil_div(m, 16) : (int64_t)ceil_div(m, ccs.tail.bm) * ceil_div(n - ccs.cols_main, ccs.tail.bn);
        }
        if (plan->lds_bytes > lds_per_cu) {
          set_error("mfma variant %d needs %d bytes of LDS, device has %d", ct.id, plan->lds_bytes, lds_per_cu);
          return GZ_ERR_UNSUPPORTED;
        }
        return GZ_OK;
      }
      if ((variant == 0 || variant == MFMA_VARIANT_STREAMK_W4 || variant == MFMA_VARIANT_STREAMK_W8) && k > 0) {   // as launch_mfma, aligned operands assumed
        StreamKPlan skp;
        const MfmaCfg* forced = variant == 0 ? nullptr : &kMfmaCfgs[variant - 1];
        if (mfma_plan_streamk(types, m, n, k, layoutA, layoutB, num_cus, forced != nullptr, forced, &skp) &&
            (forced || (size_t)skp.slots * MFMA_STREAMK_SLOT_BYTES <= ws_limit)) {
          const MfmaCfg& c = skp.cfg;
          plan->variant = c.waves_n == 4 ? MFMA_VARIANT_STREAMK_W8 : MFMA_VARIANT_STREAMK_W4;
          plan->tile_m = c.bm; plan->tile_n = c.bn; plan->tile_k = MFMA_SLAB_BYTES / es;
          plan->wave_m = c.bm / c.waves_m; plan->wave_n = c.bn / c.waves_n;
          plan->threads = c.waves_m * c.waves_n * 64;
          plan->lds_bytes = mfma_lds_bytes(c);
          plan->grid = (int64_t)skp.dp_tiles + skp.blocks;
          plan->streamk_tiles = skp.sk_tiles;
          plan->streamk_blocks = skp.blocks;
          plan->workspace_bytes = (int64_t)skp.slots * MFMA_STREAMK_SLOT_BYTES;
          if (plan->lds_bytes > lds_per_cu) {
            set_error("mfma variant %d needs %d bytes of LDS, device has %d", plan->variant, plan->lds_bytes, lds_per_cu);
            return GZ_ERR_UNSUPPORTED;
          }
          return GZ_OK;
        }
      }
      MfmaCfg c;
      MfmaSplit sp;
      MfmaColSplit cs;
      int m_first = m, n_first = n;
      const int cut = (variant == 0 && k > 0) ? mfma_resolve_cut(types, m, n, k, layoutA, layoutB, num_cus, &sp, &cs) : 0;
      if (cut == 1) {
        c = sp.main;
        m_first = sp.rows_main;
        plan->tail_rows = m - sp.rows_main;
        plan->tail_tile_m = sp.tail.bm;
        plan->tail_tile_n = sp.tail.bn;
        plan->tail_grid = (int64_t)ceil_div(m - sp.rows_main, sp.tail.bm) * ceil_div(n, sp.tail.bn);
      } else if (cut == 2) {
        c = cs.main;
        n_first = cs.cols_main;
        plan->tail_cols = n - cs.cols_main;
        if (cs.strip) {   // dot products, one wave per row, sixteen rows per work-group
          plan->tail_tile_m = 16;
          plan->tail_tile_n = plan->tail_cols;
          plan->tail_grid = ceil_div(m, 16);
        } else {
          plan->tail_tile_m = cs.tail.bm;
          plan->tail_tile_n = cs.tail.bn;
          plan->tail_grid = (int64_t)ceil_div(m, cs.tail.bm) * ceil_div(n - cs.cols_main, cs.tail.bn);
        }
      } else if (!mfma_resolve(types, m, n, k, layoutA, layoutB, variant, num_cus, &c)) {
        set_error("mfma rung: unknown variant %d", variant);
        return GZ_ERR_UNSUPPORTED;
      }
      if (variant == 0) {   // as the launcher does, with 16-byte aligned operands assumed
        int cls = mfma_shape_class(c, es, m_first, n_first, k, layoutA, layoutB);
        // (a column range of a row-major B keeps the pitch of the whole matrix: whole 16-byte pieces or not)
        if (plan->tail_cols && layoutB == GZ_ROW_MAJOR && ((int64_t)n * es) % 16 != 0) cls = MFMA_SHAPE_GENERAL;
        mfma_adjust_general(types, cls, layoutA, layoutB, &c);
      }
      plan->variant = c.id;
      plan->tile_m = c.bm; plan->tile_n = c.bn; plan->tile_k = MFMA_SLAB_BYTES / es;
      plan->wave_m = c.bm / c.waves_m; plan->wave_n = c.bn / c.waves_n;
      plan->threads = c.waves_m * c.waves_n * 64;
      plan->lds_bytes = mfma_lds_bytes(c);
      plan->grid = (int64_t)ceil_div(m_first, c.bm) * ceil_div(n_first, c.bn);
      // the ring kernel with the 16x16 instructions (whole tiles, or ragged M and N on its 256 x 256 tile): one
      // work-group per compute unit walks the tiles
      int cls_g = mfma_shape_class(c, es, m_first, n_first, k, layoutA, layoutB);
      if (plan->tail_cols && layoutB == GZ_ROW_MAJOR && ((int64_t)n * es) % 16 != 0) cls_g = MFMA_SHAPE_GENERAL;
      if (c.ring == 1 && (layoutA == GZ_ROW_MAJOR || (layoutB == GZ_ROW_MAJOR && !is_fp8(types) && types != GZ_F32F32F32)) &&
          !(types == GZ_F32F32F32 && c.waves_n != 2) &&
          (cls_g == MFMA_SHAPE_WHOLE || (cls_g == MFMA_SHAPE_RAGGED_MN && c.bm == 256)))
        plan->grid = mfma_persistent_grid(plan->grid, num_cus);
      if (plan->lds_bytes > lds_per_cu) {
        set_error("mfma variant %d needs %d bytes of LDS, device has %d", c.id, plan->lds_bytes, lds_per_cu);
        return GZ_ERR_UNSUPPORTED;
      }
      return GZ_OK;
    }
    case GZ_RUNG_SKINNY: {
      if (!skinny_supported(types, m, n, k, layoutA, layoutB)) {
        set_error("skinny rung needs a 16-bit float type, row-major A, column-major B, M <= %d and K %% %d == 0",
                  SKINNY_MAX_M, SKINNY_K_STEP);
        return GZ_ERR_UNSUPPORTED;
      }
      if (variant > 1) { set_error("skinny rung has a single variant"); return GZ_ERR_UNSUPPORTED; }
      SkinnyCfg c = skinny_resolve(m, n, k, num_cus, (unsigned long long)ws_limit);
      plan->variant = 1;
      plan->tile_m = c.mb; plan->tile_n = c.cols_per_wg;
      plan->tile_k = c.kind == SKINNY_KIND_TILE ? STREAM_TILE_K_STEP : c.kind == SKINNY_KIND_DTL ? SKINNY_DTL_K_STEP : SKINNY_K_STEP;
      plan->wave_m = c.kind == SKINNY_KIND_TILE ? 32 : c.mb; plan->wave_n = c.cols_per_wave;
      plan->threads = c.threads; plan->split_k = c.split_k; plan->lds_bytes = c.lds_bytes;
      plan->grid = (int64_t)c.grid_n * c.split_k;
      if (c.kind == SKINNY_KIND_TILE_WIDE) {   // whole rounds of the eight XCDs; a second launch adds the K parts
        const int per_round = 8 / c.split_k;
        plan->grid = (int64_t)((c.grid_n + per_round - 1) / per_round) * 8;
        plan->workspace_bytes = c.workspace_bytes;
      }
      return GZ_OK;
    }
    default: break;
  }
  set_error("unknown rung %d", rung);
  return GZ_ERR_BAD_ARG;
}

int gz_plan(int types, int64_t M, int64_t N, int64_t K, int layoutA, int layoutB, int rung, int variant, int num_cus,
            int lds_per_cu, gz_plan_t* plan) {
  return plan_impl(types, M, N, K, layoutA, layoutB, rung, variant, num_cus, lds_per_cu, ~(size_t)0, plan);
}

int gz_plan_static_scratch(int types, int64_t M, int64_t N, int64_t K, int layoutA, int layoutB, int rung, int variant,
                           int num_cus, int lds_per_cu, gz_plan_t* plan) {
  return plan_impl(types, M, N, K, layoutA, layoutB, rung, variant, num_cus, lds_per_cu,
                   (size_t)GZ_STATIC_SCRATCH_BYTES, plan);
}

const char* gz_rung_name(int rung) { return (rung >= 0 && rung < GZ_NUM_RUNGS) ? kRungNames[rung] : "auto"; }
const char* gz_types_name(int types) { return (types >= 0 && types < GZ_NUM_TYPES) ? kTypesNames[types] : "?"; }
const char* gz_last_error(void) { return g_err; }
int gz_version(void) { return 1; }

}  // extern "C"
