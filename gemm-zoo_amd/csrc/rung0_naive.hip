// Rung 0: one thread per output element, scalar loads, sequential k.
// Follows the definition of the operation in gemm-zoo
// (nvidia/kernels/naive_gemm.cuh:6-21, intel/utils/reference_kernel.hpp:12-28),
// generalised to column-major operands; the accumulator is fp32 / int32, or the 16-bit
// running sum of the reference's own kernels for the two opt-in modes.
#include "gz_common.hpp"

namespace gz {

template <int TYPES, bool A_ROW, bool B_ROW>
__global__ void __launch_bounds__(1024) naive_gemm_kernel(GemmArgs<TYPES> g) {
  const int col = threadIdx.x + blockIdx.x * blockDim.x;
  const int row = threadIdx.y + blockIdx.y * blockDim.y;
  if (row >= g.M || col >= g.N) return;

  RunningSum<TYPES> sum;
  for (int i = 0; i < g.K; i++) {
    const auto a = widen_in<TYPES>(A_ROW ? g.A[(size_t)row * g.lda + i] : g.A[(size_t)i * g.lda + row]);
    const auto b = widen_in<TYPES>(B_ROW ? g.B[(size_t)i * g.ldb + col] : g.B[(size_t)col * g.ldb + i]);
    sum.mac(a, b, i, g.K);
  }
  g.D[(size_t)row * g.ldd + col] = epilogue<TYPES>(sum.finish(g.K), g.alpha, g.beta, g.C + (size_t)row * g.ldc + col);
}

template <int TYPES> int launch_naive(const GemmArgs<TYPES>& g, int variant, hipStream_t s) {
  if (variant != 0) {
    set_error("naive rung has a single variant (got %d)", variant);
    return GZ_ERR_UNSUPPORTED;
  }
  dim3 block(32, 32, 1);  // nvidia/kernel_functors/naive_gemm.cuh:15-16
  dim3 grid(ceil_div(g.N, 32), ceil_div(g.M, 32), 1);
  if (grid.y > 65535u) {
    set_error("naive rung: M=%d needs more than 65535 block rows", g.M);
    return GZ_ERR_UNSUPPORTED;
  }
  const bool ar = g.layoutA == GZ_ROW_MAJOR, br = g.layoutB == GZ_ROW_MAJOR;
  if (ar && br) hipLaunchKernelGGL((naive_gemm_kernel<TYPES, true, true>), grid, block, 0, s, g);
  else if (ar && !br) hipLaunchKernelGGL((naive_gemm_kernel<TYPES, true, false>), grid, block, 0, s, g);
  else if (!ar && br) hipLaunchKernelGGL((naive_gemm_kernel<TYPES, false, true>), grid, block, 0, s, g);
  else hipLaunchKernelGGL((naive_gemm_kernel<TYPES, false, false>), grid, block, 0, s, g);
  GZ_HIP_TRY(hipGetLastError());
  return GZ_OK;
}

template int launch_naive<GZ_S8S8S32>(const GemmArgs<GZ_S8S8S32>&, int, hipStream_t);
template int launch_naive<GZ_BF16BF16F32>(const GemmArgs<GZ_BF16BF16F32>&, int, hipStream_t);
template int launch_naive<GZ_BF16BF16BF16>(const GemmArgs<GZ_BF16BF16BF16>&, int, hipStream_t);
template int launch_naive<GZ_F16F16F16>(const GemmArgs<GZ_F16F16F16>&, int, hipStream_t);
template int launch_naive<GZ_F32F32F32>(const GemmArgs<GZ_F32F32F32>&, int, hipStream_t);
template int launch_naive<GZ_E4M3E4M3F16>(const GemmArgs<GZ_E4M3E4M3F16>&, int, hipStream_t);
template int launch_naive<GZ_E5M2E5M2F16>(const GemmArgs<GZ_E5M2E5M2F16>&, int, hipStream_t);
template int launch_naive<GZ_BF16BF16BF16_ACC16>(const GemmArgs<GZ_BF16BF16BF16_ACC16>&, int, hipStream_t);
template int launch_naive<GZ_F16F16F16_ACC16>(const GemmArgs<GZ_F16F16F16_ACC16>&, int, hipStream_t);

}  // namespace gz
