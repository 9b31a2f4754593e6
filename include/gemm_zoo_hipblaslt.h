/*
 * gemm_zoo_hipblaslt.h -- C ABI of the vendor-library comparator (libgemmzoo_hipblaslt.so).
 *
 * The same GEMM as gemm_zoo.h through hipBLASLt with a heuristic-selected algorithm.  Reported beside the
 * ladder's numbers and used by the harness as the first-choice verifier; never part of a product result.
 *
 * Replaces utils::cublaslt_gemm (nvidia/utils/cublaslt_gemm.cuh:52-129) and the cublasLt_gemm functor
 * (nvidia/kernel_functors/cublaslt_gemm.cuh:15-125).
 */
#ifndef GEMM_ZOO_HIPBLASLT_H
#define GEMM_ZOO_HIPBLASLT_H

#include "gemm_zoo.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Plans D (M x N, row-major) = alpha * A x B + beta * C for one type bundle / layout pair; *plan owns the
 * hipBLASLt handle, descriptors and a 64 MiB workspace until gz_hipblaslt_destroy. */
int gz_hipblaslt_create(int types, int64_t M, int64_t N, int64_t K, int layoutA, int layoutB, void** plan);
int gz_hipblaslt_run(void* plan, const void* A, const void* B, const void* C, void* D, double alpha, double beta,
                     gz_stream stream);
int gz_hipblaslt_destroy(void* plan);
const char* gz_hipblaslt_last_error(void);

#ifdef __cplusplus
}
#endif
#endif
