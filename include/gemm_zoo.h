/*
 * gemm_zoo.h -- C ABI of the MI355X (gfx950) GEMM kernel ladder.
 *
 * D = alpha * (A x B) + beta * C   with A: M x K, B: K x N, C and D: M x N.
 *
 * All matrix pointers are DEVICE pointers owned by the caller.  The typed entry
 * points and gz_gemm take packed matrices (the leading dimension equals the
 * contiguous extent); gz_gemm_ld takes the four leading dimensions.  C and D are
 * always row-major.  A and B carry a layout flag each.  When beta == 0, C is
 * never read and may be NULL.  D must not overlap A or B.  Calls are
 * asynchronous on `stream` (a hipStream_t, NULL = the default stream); the
 * caller synchronises.  M, N, K and the leading dimensions stay below 2^31; the
 * matrices themselves may hold 2^31 elements and more (the reference indexes
 * with std::size_t, nvidia/utils/benchmark.cuh:17, nvidia/kernels/naive_gemm.cuh:8).
 *
 * Every function returns a gz_status; nothing exits the process or throws.
 * gz_last_error() gives the message of the calling thread's last failure.
 *
 * What each entry point stands in for in gemm-zoo (paths relative to its tree):
 *   typed GEMM entry points  <-  the kernel functors' operator()
 *       nvidia/kernel_functors/bf16_mma_gemm.cuh:51-63   (bf16 x bf16 -> f32)
 *       nvidia/kernel_functors/fp16_mma_gemm.cuh:16-70   (fp16 x fp16 -> fp16)
 *       intel/xe_gemm_s8_s8_s32_m8k16.hpp:12-40          (s8 x s8 -> s32)
 *       intel/xe_gemm_bf16_bf16_f32_m8k16.hpp:12-47      (bf16 x bf16 -> f32)
 *       intel/xe_gemm_bf16_bf16_bf16_m8k16.hpp:12-47     (bf16 x bf16 -> bf16)
 *       nvidia/kernel_functors/naive_gemm.cuh:12-31, generic_gemm.cuh:14-41,
 *       smem_tiled_gemm.cuh:14-51, rmem_tiled_gemm.cuh:15-55,
 *       double_buffered_gemm.cuh:15-57, async_buffered_gemm.cuh:16-58 (ladder rungs; the reference's
 *       drivers for these run fp32 x fp32 -> fp32, e.g. nvidia/bench/bench_naive.cu:9-17: gz_gemm_f32f32f32)
 *   gz_plan                   <-  the functors' constructors (grid/block/LDS
 *       computation and shape checks), e.g. nvidia/kernel_functors/bf16_mma_gemm.cuh:18-49
 *   gz_fill                   <-  utils::populate_with_random nvidia/utils/fill_data.cuh:33-49,
 *                                 test::populate_with_random intel/test/utils.hpp:27-45
 *   gz_compare                <-  utils::compare_results nvidia/utils/compare.cuh:32-47,
 *                                 test::compare_results intel/test/utils.hpp:47-73
 *
 * Arithmetic contract (what the parity tests hold the kernels to):
 *   s8s8s32     : int32 accumulate, D = alpha*acc + beta*C in wrapping int32.
 *   bf16bf16f32 : fp32 accumulate, v = acc*alpha; if (beta != 0) v += beta*C; each
 *                 operation rounded to fp32 (no fused multiply-add in the epilogue).
 *   bf16bf16bf16, f16f16f16 : fp32 accumulate, then the same epilogue evaluated in the
 *                 16-bit output type: v = T(acc); v = T(v*alpha); if (beta != 0)
 *                 v = T(v + T(beta*C)) -- nvidia/kernels/generic_gemm.cuh:53-58.
 *                 alpha and beta are rounded to the output type first.
 *   e4m3e4m3f16, e5m2e5m2f16 : inputs are OCP 8-bit floats (e4m3: bias 7, no infinities, 0x7f/0xff NaN, largest
 *                 448; e5m2: the upper byte of an IEEE half); every product is exact in fp32; fp32 accumulate;
 *                 epilogue in fp16 as for f16f16f16 (the reference's checker computes these types in float,
 *                 nvidia/kernels/generic_gemm.cuh:10-13,53-58).
 *   bf16bf16bf16_acc16, f16f16f16_acc16 : opt-in modes with the reference kernels' 16-bit accumulator.  K is cut into
 *                 chunks of 16 (bf16: one DPAS of intel/kernels/xe_gemm_bf16_bf16_bf16_m8k16.hpp:88-97, whose C
 *                 operand is bf16) or 8 (fp16: one mma.sync.m16n8k8.f16.f16.f16.f16 of
 *                 nvidia/kernels/sm_80/fp16_mma_gemm.cuh:179) consecutive k; a chunk's products are summed in fp32
 *                 starting from zero, and the 16-bit running sum becomes T(fp32(sum16 + chunk)).  Epilogue bf16:
 *                 T(T(alpha*acc) + T(beta*C)) (xe_gemm_bf16_bf16_bf16_m8k16.hpp:104-107); fp16: one fused
 *                 multiply-add in half precision, fma(alpha, acc, T(beta*C)) (fp16_mma_gemm.cuh:279-290).  With
 *                 beta == 0, C is not read and the addend is +0.  How the hardware of the reference sums inside
 *                 one instruction is not published; the chunking and the 16-bit running sum are what is modelled.
 *   f32f32f32   : fp32 accumulate in k order with each product fused into the sum (fma), which is what the
 *                 reference's `acc += a * b` (nvidia/kernels/naive_gemm.cuh:16-19) compiles to; epilogue as
 *                 bf16bf16f32.  The MFMA rung uses the full-precision v_mfma_f32_32x32x2_f32, not a tf32 mode.
 */
#ifndef GEMM_ZOO_H
#define GEMM_ZOO_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum gz_status {
  GZ_OK = 0,
  GZ_ERR_BAD_ARG = 1,     /* null pointer, negative size, unknown enum value      */
  GZ_ERR_UNSUPPORTED = 2, /* valid request this rung / variant cannot serve       */
  GZ_ERR_HIP = 3,         /* a HIP runtime call failed; see gz_last_error()       */
  GZ_ERR_MISMATCH = 4     /* gz_compare found differing elements                  */
} gz_status;

typedef enum gz_layout { GZ_ROW_MAJOR = 0, GZ_COL_MAJOR = 1 } gz_layout;

typedef enum gz_types {
  GZ_S8S8S32 = 0,
  GZ_BF16BF16F32 = 1,
  GZ_BF16BF16BF16 = 2,
  GZ_F16F16F16 = 3,
  GZ_F32F32F32 = 4,
  GZ_E4M3E4M3F16 = 5, /* OCP fp8 e4m3 (finite-only, __nv_fp8_e4m3's format) x e4m3 -> fp16 */
  GZ_E5M2E5M2F16 = 6, /* OCP fp8 e5m2 (__nv_fp8_e5m2's format) x e5m2 -> fp16            */
  GZ_BF16BF16BF16_ACC16 = 7, /* bf16 x bf16 -> bf16 with a bf16 running sum, chunks of 16 k */
  GZ_F16F16F16_ACC16 = 8,    /* fp16 x fp16 -> fp16 with an fp16 running sum, chunks of 8 k  */
  GZ_NUM_TYPES = 9
} gz_types;

/* The ladder.  GZ_RUNG_AUTO lets the launcher pick (MFMA, or the weight-streaming
 * kernel for skinny M).                                                            */
typedef enum gz_rung {
  GZ_RUNG_AUTO = -1,
  GZ_RUNG_NAIVE = 0,           /* one thread per output, scalar loads              */
  GZ_RUNG_COALESCED = 1,       /* layout-aware lane mapping, 128-bit global loads  */
  GZ_RUNG_LDS_TILED = 2,       /* LDS tiles with bank-conflict-free padding        */
  GZ_RUNG_DOUBLE_BUFFERED = 3, /* global->LDS prefetch overlapped with compute     */
  GZ_RUNG_MFMA = 4,            /* wavefront-level matrix-core kernel               */
  GZ_RUNG_SKINNY = 5,          /* weight-streaming kernels for M <= 128            */
  GZ_NUM_RUNGS = 6
} gz_rung;

typedef void* gz_stream; /* hipStream_t */

/* Launch geometry the launcher chose for a problem (host-only computation). */
typedef struct gz_plan_t {
  int32_t rung;        /* resolved rung (never GZ_RUNG_AUTO)                   */
  int32_t variant;     /* resolved tile-config id within the rung              */
  int32_t tile_m, tile_n, tile_k;
  int32_t wave_m, wave_n;      /* per-wavefront sub-tile (0 if not applicable) */
  int32_t threads;             /* work-group size                              */
  int32_t lds_bytes;           /* static + dynamic LDS per work-group          */
  int64_t grid;                /* number of work-groups                        */
  int32_t split_k;             /* >1: partial sums reduced in a second pass    */
  int32_t vector_bytes_a, vector_bytes_b; /* widest aligned global access used */
  /* MFMA rung, launcher's choice only: when the tiles would leave a mostly empty last round of the compute
   * units, the last tail_rows rows of the problem run in a second launch with their own tile (0: one launch).
   * rung, tile_*, grid above then describe the first launch (M - tail_rows rows).                          */
  int32_t tail_rows;
  int32_t tail_tile_m, tail_tile_n;
  int64_t tail_grid;
  /* The same for columns: N a few columns past a multiple of 256 would put them into a tile column of their own
   * that costs as much as a whole one; the last tail_cols columns then run in a second launch (tail_tile_*,
   * tail_grid describe it; 0: no such split; never together with tail_rows).                                  */
  int32_t tail_cols;
  /* MFMA rung, stream-K (variants 7 and 8, and the launcher's choice where its estimate prefers it): the 256x256
   * tiles past the last whole round of the compute units, streamk_tiles of them, have their K slabs dealt in equal
   * contiguous runs to streamk_blocks work-groups of the same launch (grid = whole tiles + streamk_blocks); every
   * run leaves partial sums in a workspace of workspace_bytes that the caller never sees, and a second launch
   * adds a tile's pieces in a fixed order (results do not depend on timing).  0: no such decomposition.       */
  int32_t streamk_tiles, streamk_blocks;
  int64_t workspace_bytes;
} gz_plan_t;

/* variant: 0 = launcher's choice; other values select a tile configuration of the rung (1 .. gz_variant_count).
 * MFMA rung: 1 256x256 on four waves, 2 on eight, 3 128x128, 4 256x128 (register-staged or compiler-scheduled
 * direct-to-LDS kernels, any shape and layout); 5 / 6 the hand-scheduled 256x256 ring kernel on four / eight waves
 * wherever the problem allows it (row-major A, whole K slabs, 16-byte aligned rows; otherwise the kernel of 1 / 2);
 * 7 / 8 the same with the stream-K decomposition; 9 / 10 as 5 / 6 with one work-group per tile instead of one per
 * compute unit; 11 the ring kernel on 128x128 tiles, two work-groups per compute unit (int8, the 16-bit types and
 * fp32; otherwise the kernel of 3); 12 the register-staged kernel on 64x64 tiles (four waves; two for 8-bit
 * elements).                                                                                                   */
int gz_gemm_s8s8s32(const int8_t* A, const int8_t* B, const int32_t* C, int32_t* D,
                    int64_t M, int64_t N, int64_t K, int layoutA, int layoutB,
                    int32_t alpha, int32_t beta, int rung, int variant, gz_stream stream);

int gz_gemm_bf16bf16f32(const uint16_t* A, const uint16_t* B, const float* C, float* D,
                        int64_t M, int64_t N, int64_t K, int layoutA, int layoutB,
                        float alpha, float beta, int rung, int variant, gz_stream stream);

int gz_gemm_bf16bf16bf16(const uint16_t* A, const uint16_t* B, const uint16_t* C, uint16_t* D,
                         int64_t M, int64_t N, int64_t K, int layoutA, int layoutB,
                         float alpha, float beta, int rung, int variant, gz_stream stream);

int gz_gemm_f16f16f16(const uint16_t* A, const uint16_t* B, const uint16_t* C, uint16_t* D,
                      int64_t M, int64_t N, int64_t K, int layoutA, int layoutB,
                      float alpha, float beta, int rung, int variant, gz_stream stream);

int gz_gemm_f32f32f32(const float* A, const float* B, const float* C, float* D,
                      int64_t M, int64_t N, int64_t K, int layoutA, int layoutB,
                      float alpha, float beta, int rung, int variant, gz_stream stream);

/* fp8 inputs (one byte per element, raw bit patterns), fp16 output: the bundles of the reference's
 * cublasLt_gemm<__nv_fp8_e4m3, __half> / <__nv_fp8_e5m2, __half> (nvidia/kernel_functors/cublaslt_gemm.cuh,
 * nvidia/bench/bench_cublaslt_e4m3.cu:6-21, bench_cublaslt_e5m2.cu:6-21), which the reference only runs through
 * cuBLASLt; here they have kernels of their own on every rung.                                              */
int gz_gemm_e4m3e4m3f16(const uint8_t* A, const uint8_t* B, const uint16_t* C, uint16_t* D,
                        int64_t M, int64_t N, int64_t K, int layoutA, int layoutB,
                        float alpha, float beta, int rung, int variant, gz_stream stream);

int gz_gemm_e5m2e5m2f16(const uint8_t* A, const uint8_t* B, const uint16_t* C, uint16_t* D,
                        int64_t M, int64_t N, int64_t K, int layoutA, int layoutB,
                        float alpha, float beta, int rung, int variant, gz_stream stream);

/* The reference kernels' own 16-bit accumulators as opt-in modes (see the arithmetic contract above): the bf16
 * accumulator of intel::gemm_bf16_bf16_bf16_m8k16 (intel/kernels/xe_gemm_bf16_bf16_bf16_m8k16.hpp:88-107) and the
 * fp16 accumulator of nvidia::kernels::sm80::fp16_mma_gemm (nvidia/kernels/sm_80/fp16_mma_gemm.cuh:179,279-290).
 * Served by the naive, coalesced, LDS-tiled, double-buffered and MFMA rungs; the weight-streaming rung refuses.  */
int gz_gemm_bf16bf16bf16_acc16(const uint16_t* A, const uint16_t* B, const uint16_t* C, uint16_t* D,
                               int64_t M, int64_t N, int64_t K, int layoutA, int layoutB,
                               float alpha, float beta, int rung, int variant, gz_stream stream);

int gz_gemm_f16f16f16_acc16(const uint16_t* A, const uint16_t* B, const uint16_t* C, uint16_t* D,
                            int64_t M, int64_t N, int64_t K, int layoutA, int layoutB,
                            float alpha, float beta, int rung, int variant, gz_stream stream);

/* Type-erased form of the typed entry points above (alpha/beta as double; for s8s8s32 they must be
 * integral).                                                                         */
int gz_gemm(int types, const void* A, const void* B, const void* C, void* D,
            int64_t M, int64_t N, int64_t K, int layoutA, int layoutB,
            double alpha, double beta, int rung, int variant, gz_stream stream);

/* gz_gemm on matrices with leading dimensions, in elements, as nvidia::kernels::generic_gemm takes them
 * (nvidia/kernels/generic_gemm.cuh:6-8; its functor passes the packed values, nvidia/kernel_functors/generic_gemm.cuh:30-32):
 * lda between consecutive rows of a row-major A (at least K) or columns of a column-major one (at least M), ldb between
 * the K rows of a row-major B (at least N) or the columns of a column-major one (at least K), ldc / ldd between the rows
 * of C / D (at least N).  0 stands for the packed value.  Every rung takes them; the direct-to-LDS kernels of the MFMA
 * rung and the weight-streaming rung need leading dimensions that are whole 16-byte pieces (the launcher's choice falls
 * back to the register-staged kernels otherwise, an explicit GZ_RUNG_SKINNY returns GZ_ERR_UNSUPPORTED).            */
int gz_gemm_ld(int types, const void* A, int64_t lda, const void* B, int64_t ldb, const void* C, int64_t ldc,
               void* D, int64_t ldd, int64_t M, int64_t N, int64_t K, int layoutA, int layoutB,
               double alpha, double beta, int rung, int variant, gz_stream stream);

/* gz_gemm for callers that cannot allocate device memory: code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc.  It has no counterpart in the reference.  Same arguments and the same results,
 * bit for bit, as gz_gemm.  The one difference is where a stream-K launch (see gz_plan_t) keeps its partial sums:
 * not in the library's pool, which hipMalloc grows on demand, but in a buffer of GZ_STATIC_SCRATCH_BYTES (384
 * slots of 256 x 256 accumulators) that is part of the library's device image, so that every GPU the library runs
 * on holds its own copy until the process ends.  This entry point never allocates or frees.  A launch that would
 * need more than that does not arise under the launcher's own choice (variant 0): there the launcher keeps to plans
 * that fit (gz_plan_static_scratch reports them; they may differ from gz_plan's where gz_plan's workspace_bytes exceeds
 * the buffer, and then the results agree with gz_gemm's within the type's tolerance instead of bit for bit).  An
 * explicit stream-K variant (7, 8) that needs more returns GZ_ERR_UNSUPPORTED with both sizes in gz_last_error(); the
 * variants without stream-K never need any.  The buffer keeps the last call's contents;
 * nothing in it has to start at zero, every slot is written before it is read.  All calls on one GPU share it:
 * calls that overlap in time on one GPU (two streams, two host threads) race on it and must be serialised by the
 * caller.                                                                                                       */
#define GZ_STATIC_SCRATCH_BYTES (96ll << 20)
int gz_gemm_static_scratch(int types, const void* A, const void* B, const void* C, void* D,
                           int64_t M, int64_t N, int64_t K, int layoutA, int layoutB,
                           double alpha, double beta, int rung, int variant, gz_stream stream);

/* Host-only: resolve rung/variant and compute the launch geometry for a problem on a
 * device with `num_cus` compute units and `lds_per_cu` bytes of LDS (0 = MI355X: 256 CUs,
 * 160 KiB).  Performs the same argument checks as the GEMM entry points.  The GEMM entry
 * points size their launches for the compute units of the device they run on
 * (hipDeviceAttributeMultiprocessorCount of the current device): pass that count here
 * to get the geometry they will choose there.                                        */
int gz_plan(int types, int64_t M, int64_t N, int64_t K, int layoutA, int layoutB,
            int rung, int variant, int num_cus, int lds_per_cu, gz_plan_t* plan);

/* The same for gz_gemm_static_scratch: the launcher's choice (variant 0) keeps to plans whose workspace_bytes fit
 * GZ_STATIC_SCRATCH_BYTES.  No counterpart in the reference.                                                    */
int gz_plan_static_scratch(int types, int64_t M, int64_t N, int64_t K, int layoutA, int layoutB,
                           int rung, int variant, int num_cus, int lds_per_cu, gz_plan_t* plan);

/* The two device properties the functor constructors plan with (what nvidia/utils/benchmark.cuh:20-24 reads
 * into cudaDeviceProp for every functor): compute units and LDS bytes per compute unit of the device that is
 * current on the calling thread.  Either pointer may be NULL.                          */
int gz_device_props(int32_t* num_cus, int32_t* lds_per_cu);

int gz_variant_count(int types, int rung);
const char* gz_rung_name(int rung);
const char* gz_types_name(int types);

/* Seeded device fill: element i of `dst` is a pure function of (seed, i) through
 * Philox4x32-10 with counter = i and key = seed.
 *   dtype: 0 int8, 1 bf16, 2 fp16, 3 fp32, 4 int32, 5 fp8 e4m3, 6 fp8 e5m2 (round to nearest even,
 *          saturating to the largest finite value)
 *   kind : 0 integers uniform in [-128,127]   1 N(0,1)*scale   2 U(-1,1)*scale
 *          3 small integers in {-1,0,1} (exactly representable partial sums)      */
int gz_fill(void* dst, int64_t count, int dtype, int kind, float scale, uint64_t seed,
            gz_stream stream);

/* Element-wise compare of two device arrays.  abs_threshold == 0 demands exact equality
 * of the stored values; otherwise |out - ref| > abs_threshold counts as different.
 * Synchronises `stream`.  *num_different (host memory, may be NULL) receives the count.
 * Returns GZ_ERR_MISMATCH if any element differs.
 *   dtype as in gz_fill (0..4; 8-bit floats are inputs only).                        */
int gz_compare(const void* out, const void* ref, int64_t count, int dtype,
               float abs_threshold, int64_t* num_different, gz_stream stream);

/* As gz_compare with a mixed bound: an element differs when |out - ref| > abs_threshold + rel_threshold * |ref|
 * (both zero: exact equality).  For 16-bit outputs, whose rounding step grows with the value, an absolute
 * bound alone (nvidia/utils/compare.cuh:19 uses 0.5) is either too loose or too tight. */
int gz_compare_rel(const void* out, const void* ref, int64_t count, int dtype, float abs_threshold,
                   float rel_threshold, int64_t* num_different, gz_stream stream);

const char* gz_last_error(void);
int gz_version(void);

#ifdef __cplusplus
}
#endif
#endif /* GEMM_ZOO_H */
