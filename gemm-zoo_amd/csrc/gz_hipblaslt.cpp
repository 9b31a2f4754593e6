// Vendor-library comparator: the same GEMM through hipBLASLt (heuristic-selected algorithm).
//
// Built into its own shared object (libgemmzoo_hipblaslt.so) so that the product library depends on the
// HIP runtime only.  It is "reported alongside" in the benchmarks and is itself checked against the CPU
// oracle in the tests; it is never used to produce a result of the product.
//
// Stands in for utils::cublaslt_gemm (nvidia/utils/cublaslt_gemm.cuh:52-129) and the cublasLt_gemm functor
// (nvidia/kernel_functors/cublaslt_gemm.cuh:15-125).  Unlike those, the operand orders are set explicitly:
// the row-major product D = A x B is computed as the column-major product D^T = B^T x A^T, every handle,
// descriptor and the workspace are released by gz_hipblaslt_destroy, and failures come back as codes.
#include <hip/hip_runtime.h>
#include <hipblaslt/hipblaslt.h>
#include <stdarg.h>
#include <stdint.h>
#include <stdio.h>

#include "../../include/gemm_zoo.h"

namespace {

thread_local char g_err[512] = "";
void set_err(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
}

struct Plan {
  hipblasLtHandle_t handle = nullptr;
  hipblasLtMatmulDesc_t desc = nullptr;
  hipblasLtMatrixLayout_t la = nullptr, lb = nullptr, lc = nullptr, ld = nullptr;
  hipblasLtMatmulPreference_t pref = nullptr;
  hipblasLtMatmulHeuristicResult_t heur{};
  void* workspace = nullptr;
  size_t workspace_bytes = 0;
  int types = 0;
  ~Plan() {
    if (pref) hipblasLtMatmulPreferenceDestroy(pref);
    if (la) hipblasLtMatrixLayoutDestroy(la);
    if (lb) hipblasLtMatrixLayoutDestroy(lb);
    if (lc) hipblasLtMatrixLayoutDestroy(lc);
    if (ld) hipblasLtMatrixLayoutDestroy(ld);
    if (desc) hipblasLtMatmulDescDestroy(desc);
    if (handle) hipblasLtDestroy(handle);
    if (workspace) (void)hipFree(workspace);
  }
};

#define LT_TRY(expr)                                                            \
  do {                                                                          \
    hipblasStatus_t _s = (expr);                                                \
    if (_s != HIPBLAS_STATUS_SUCCESS) {                                         \
      set_err("hipBLASLt status %d in %s", (int)_s, #expr);                     \
      delete p;                                                                 \
      return GZ_ERR_HIP;                                                        \
    }                                                                           \
  } while (0)

}  // namespace

extern "C" {

const char* gz_hipblaslt_last_error(void) { return g_err; }

// Plans D(MxN, row-major) = alpha * A x B + beta * C for one type bundle and layout pair.
int gz_hipblaslt_create(int types, int64_t M, int64_t N, int64_t K, int layoutA, int layoutB, void** plan_out) {
  if (!plan_out || types < 0 || types >= GZ_NUM_TYPES || M <= 0 || N <= 0 || K <= 0 || (layoutA | layoutB) & ~1) {
    set_err("gz_hipblaslt_create: bad argument");
    return GZ_ERR_BAD_ARG;
  }
  if (types == GZ_BF16BF16BF16_ACC16 || types == GZ_F16F16F16_ACC16) {
    set_err("gz_hipblaslt_create: the library has no 16-bit accumulation");
    return GZ_ERR_UNSUPPORTED;
  }
  hipDataType in_t, out_t, scale_t;
  hipblasComputeType_t comp;
  switch (types) {
    case GZ_S8S8S32: in_t = HIP_R_8I; out_t = HIP_R_32I; scale_t = HIP_R_32I; comp = HIPBLAS_COMPUTE_32I; break;
    case GZ_BF16BF16F32: in_t = HIP_R_16BF; out_t = HIP_R_32F; scale_t = HIP_R_32F; comp = HIPBLAS_COMPUTE_32F; break;
    case GZ_BF16BF16BF16: in_t = HIP_R_16BF; out_t = HIP_R_16BF; scale_t = HIP_R_32F; comp = HIPBLAS_COMPUTE_32F; break;
    case GZ_E4M3E4M3F16: in_t = HIP_R_8F_E4M3; out_t = HIP_R_16F; scale_t = HIP_R_32F; comp = HIPBLAS_COMPUTE_32F; break;
    case GZ_E5M2E5M2F16: in_t = HIP_R_8F_E5M2; out_t = HIP_R_16F; scale_t = HIP_R_32F; comp = HIPBLAS_COMPUTE_32F; break;
    case GZ_F32F32F32: in_t = HIP_R_32F; out_t = HIP_R_32F; scale_t = HIP_R_32F; comp = HIPBLAS_COMPUTE_32F; break;
    default: in_t = HIP_R_16F; out_t = HIP_R_16F; scale_t = HIP_R_32F; comp = HIPBLAS_COMPUTE_32F; break;
  }
  Plan* p = new Plan;
  p->types = types;
  LT_TRY(hipblasLtCreate(&p->handle));
  LT_TRY(hipblasLtMatmulDescCreate(&p->desc, comp, scale_t));
  // column-major view: first operand is our B, second our A
  const hipblasOperation_t op_first = layoutB == GZ_ROW_MAJOR ? HIPBLAS_OP_N : HIPBLAS_OP_T;
  const hipblasOperation_t op_second = layoutA == GZ_ROW_MAJOR ? HIPBLAS_OP_N : HIPBLAS_OP_T;
  LT_TRY(hipblasLtMatmulDescSetAttribute(p->desc, HIPBLASLT_MATMUL_DESC_TRANSA, &op_first, sizeof(op_first)));
  LT_TRY(hipblasLtMatmulDescSetAttribute(p->desc, HIPBLASLT_MATMUL_DESC_TRANSB, &op_second, sizeof(op_second)));
  // memory of B: row-major KxN == column-major NxK (ld N); column-major (N lines of K) == column-major KxN (ld K)
  if (layoutB == GZ_ROW_MAJOR) LT_TRY(hipblasLtMatrixLayoutCreate(&p->la, in_t, N, K, N));
  else LT_TRY(hipblasLtMatrixLayoutCreate(&p->la, in_t, K, N, K));
  // memory of A: row-major MxK == column-major KxM (ld K); column-major == column-major MxK (ld M)
  if (layoutA == GZ_ROW_MAJOR) LT_TRY(hipblasLtMatrixLayoutCreate(&p->lb, in_t, K, M, K));
  else LT_TRY(hipblasLtMatrixLayoutCreate(&p->lb, in_t, M, K, M));
  LT_TRY(hipblasLtMatrixLayoutCreate(&p->lc, out_t, N, M, N));
  LT_TRY(hipblasLtMatrixLayoutCreate(&p->ld, out_t, N, M, N));
  LT_TRY(hipblasLtMatmulPreferenceCreate(&p->pref));
  p->workspace_bytes = 64u << 20;
  if (hipMalloc(&p->workspace, p->workspace_bytes) != hipSuccess) {
    set_err("workspace allocation failed");
    delete p;
    return GZ_ERR_HIP;
  }
  LT_TRY(hipblasLtMatmulPreferenceSetAttribute(p->pref, HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES, &p->workspace_bytes,
                                               sizeof(p->workspace_bytes)));
  int found = 0;
  LT_TRY(hipblasLtMatmulAlgoGetHeuristic(p->handle, p->desc, p->la, p->lb, p->lc, p->ld, p->pref, 1, &p->heur, &found));
  if (found == 0) {
    set_err("hipBLASLt has no algorithm for this problem");
    delete p;
    return GZ_ERR_UNSUPPORTED;
  }
  *plan_out = p;
  return GZ_OK;
}

int gz_hipblaslt_run(void* plan, const void* A, const void* B, const void* C, void* D, double alpha, double beta,
                     gz_stream stream) {
  Plan* p = static_cast<Plan*>(plan);
  if (!p || !A || !B || !D) {
    set_err("gz_hipblaslt_run: bad argument");
    return GZ_ERR_BAD_ARG;
  }
  float fa = (float)alpha, fb = (float)beta;
  int32_t ia = (int32_t)alpha, ib = (int32_t)beta;
  const void* pa = p->types == GZ_S8S8S32 ? (const void*)&ia : (const void*)&fa;
  const void* pb = p->types == GZ_S8S8S32 ? (const void*)&ib : (const void*)&fb;
  const void* c_arg = C ? C : D;  // beta == 0: the library still wants a valid pointer
  hipblasStatus_t s = hipblasLtMatmul(p->handle, p->desc, pa, B, p->la, A, p->lb, pb, c_arg, p->lc, D, p->ld,
                                      &p->heur.algo, p->workspace, p->workspace_bytes, static_cast<hipStream_t>(stream));
  if (s != HIPBLAS_STATUS_SUCCESS) {
    set_err("hipblasLtMatmul status %d", (int)s);
    return GZ_ERR_HIP;
  }
  return GZ_OK;
}

int gz_hipblaslt_destroy(void* plan) {
  delete static_cast<Plan*>(plan);
  return GZ_OK;
}

}  // extern "C"
