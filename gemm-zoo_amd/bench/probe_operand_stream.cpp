// What the operand stream of the 256 x 256 tile kernel costs beside the matrix instructions, without the rest of
// the kernel: the access pattern of a bf16 4096^3 launch of mfma_ring16_kernel (256 work-groups, one tile each; per
// 128-byte K slab every wave copies 8 x 1 KiB of A rows and 8 x 1 KiB of B rows straight into a ring of LDS buffers,
// three half-slab groups in flight) and its MFMAs (64 v_mfma_f32_16x16x32_bf16 per wave and K step on 64 accumulator
// blocks), each alone and together.  No LDS reads, no barriers, operands of the MFMAs held in registers.
//
//     gemm-zoo_amd/bench/bin/probe_operand_stream [settle launches = 1500] [timed launches = 200]
//
// prints microseconds per launch (1 GiB into the compute units, 137 GFLOP) for: the copies alone
// (global_load_lds_dwordx4 and buffer_load_dwordx4 ... lds), the MFMAs alone, both together on four waves, with the
// copies issued in pairs, and on eight waves (two per SIMD, half the accumulators and copies each).  With small launch
// counts (`probe_operand_stream 2 4`) it is short enough for a counter run, where the cycles per launch say whether
// a difference in time is stall cycles or clock.
#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <type_traits>

#define CHECK(x)                                                                      \
  do {                                                                                \
    hipError_t e_ = (x);                                                              \
    if (e_ != hipSuccess) {                                                           \
      std::fprintf(stderr, "%s: %s\n", #x, hipGetErrorString(e_));                    \
      std::exit(1);                                                                   \
    }                                                                                 \
  } while (0)

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

template <int N, class F, int I = 0> __device__ __forceinline__ void sfor(F&& f) {
  if constexpr (I < N) {
    f(std::integral_constant<int, I>{});
    sfor<N, F, I + 1>(static_cast<F&&>(f));
  }
}
template <int OFF> __device__ __forceinline__ void cp_global(uint32_t voff, const char* base) {
  asm volatile("global_load_lds_dwordx4 %0, %1 offset:%2" : : "v"(voff), "s"(base), "i"(OFF) : "memory");
}
template <int OFF> __device__ __forceinline__ void cp_buffer(uint32_t voff, u32x4 srd, uint32_t soff) {
  asm volatile("buffer_load_dwordx4 %0, %1, %2 offen offset:%3 lds" : : "v"(voff), "s"(srd), "s"(soff), "i"(OFF) : "memory");
}
__device__ __forceinline__ void set_m0(uint32_t v) { asm volatile("s_mov_b32 m0, %0" : : "s"(v) : "memory"); }
__device__ __forceinline__ void mfma(f32x4& c, const u32x4& a, const u32x4& b) {
  asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
}

constexpr int LDS_BYTES = 5 * 32768;
enum { COPY_NONE = 0, COPY_GLOBAL = 1, COPY_BUFFER = 2 };

// MFMAS: with the matrix instructions; COPY: which copy instruction; NWV waves; PAIR: copies issued two at a time
template <bool MFMAS, int COPY, int NWV, bool PAIR>
__global__ void __launch_bounds__(NWV * 64) probe_kernel(const char* A, const char* B, int k_bytes, int nslab, float* sink) {
  extern __shared__ __attribute__((aligned(1024))) char lds[];
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  // 16 x 16 tiles, a band of 4 x 8 of them per XCD (work-groups are dealt to the XCDs in turn)
  const int xcd = blockIdx.x % 8, i = blockIdx.x / 8;
  const int tm = (xcd / 2) * 4 + i / 8, tn = (xcd % 2) * 8 + i % 8;
  const size_t ld = (size_t)k_bytes;
  const char* a_tile = A + (size_t)tm * 256 * ld;
  const char* b_tile = B + (size_t)tn * 256 * ld;
  constexpr int NCPY = 32 / NWV, HALF = NCPY / 2;   // copies per wave and K step: A rows, then B rows
  constexpr int NACC = 256 / NWV;                   // accumulator blocks = MFMAs per wave and K step
  constexpr int WAVE_LDS = 16384 / NWV;
  const int ci = lane >> 3, cs = lane & 7;
  uint32_t voff[2][HALF];
#pragma unroll
  for (int par = 0; par < 2; par++)
#pragma unroll
    for (int t = 0; t < HALF; t++) {
      const int r = 16 * (wave * HALF + t) + 8 * par + ci;
      const uint32_t at = (uint32_t)((size_t)r * ld + (size_t)((cs ^ ci ^ par) * 16));
      voff[par][t] = COPY == COPY_BUFFER ? at - t * 1024 : at - (t - 2) * 1024 + 4096;
    }
  const uint32_t lds_base = (uint32_t)(uintptr_t)lds;
  u32x4 srd_a, srd_b;
  {
    const uint64_t pa = (uint64_t)a_tile, pb = (uint64_t)b_tile;
    srd_a = u32x4{(uint32_t)pa, (uint32_t)(pa >> 32) & 0xffff, 0xffffffffu, 0x00020000u};
    srd_b = u32x4{(uint32_t)pb, (uint32_t)(pb >> 32) & 0xffff, 0xffffffffu, 0x00020000u};
  }
#pragma unroll
  for (int e = 0; e < 4; e++) {
    srd_a[e] = __builtin_amdgcn_readfirstlane(srd_a[e]);
    srd_b[e] = __builtin_amdgcn_readfirstlane(srd_b[e]);
  }
  f32x4 acc[NACC];
#pragma unroll
  for (int q = 0; q < NACC; q++) acc[q] = f32x4{0, 0, 0, 0};
  u32x4 fa[8], fb[8];
#pragma unroll
  for (int q = 0; q < 8; q++) {   // bf16 pairs with varied mantissas and signs, magnitude about 1
    uint32_t h = (uint32_t)(lane * 2654435761u + q * 40503u + blockIdx.x * 97u);
#pragma unroll
    for (int e = 0; e < 4; e++) {
      h = h * 1664525u + 1013904223u;
      fa[q][e] = (h & 0x807f807fu) | 0x3f003f00u;
      h = h * 1664525u + 1013904223u;
      fb[q][e] = (h & 0x807f807fu) | 0x3f003f00u;
    }
  }
  auto step = [&](auto par_c, int c) {   // copy group c: the rows of parity c & 1 of slab c / 2
    constexpr int par = decltype(par_c)::value;
    const int st = c % 5;
    const uint32_t koff = (uint32_t)(c >> 1) * 128;
    const char* as = a_tile + koff - 4096;
    const char* bs = b_tile + koff - 4096;
    auto do_copy = [&](auto t_c) {
      constexpr int T = decltype(t_c)::value, TT = T % HALF;
      const uint32_t dst = lds_base + st * 32768 + (T < HALF ? 0 : 16384) + wave * WAVE_LDS;
      if constexpr (COPY == COPY_GLOBAL) {
        if constexpr (TT == 0) set_m0(dst + 2048);
        cp_global<(TT - 2) * 1024>(voff[par][TT], T < HALF ? as : bs);
      } else if constexpr (COPY == COPY_BUFFER) {
        if constexpr (TT == 0) set_m0(dst);
        cp_buffer<TT * 1024>(voff[par][TT], T < HALF ? srd_a : srd_b, koff);
      }
    };
    constexpr int CPE = NACC / NCPY;   // MFMAs per copy
    sfor<NACC>([&](auto q_c) {
      constexpr int Q = decltype(q_c)::value;
      if constexpr (MFMAS) mfma(acc[Q], fb[Q % 8], fa[(Q / 8) % 8]);
      if constexpr (!PAIR) {
        if constexpr (Q % CPE == CPE - 1) do_copy(std::integral_constant<int, Q / CPE>{});
      } else if constexpr (Q % (2 * CPE) == 2 * CPE - 1) {
        do_copy(std::integral_constant<int, 2 * (Q / (2 * CPE))>{});
        do_copy(std::integral_constant<int, 2 * (Q / (2 * CPE)) + 1>{});
      }
    });
    if constexpr (COPY != COPY_NONE) asm volatile("s_waitcnt vmcnt(%0)" : : "i"(3 * NCPY) : "memory");
  };
  for (int c = 0; c < 2 * nslab; c += 2) {
    step(std::integral_constant<int, 0>{}, c);
    step(std::integral_constant<int, 1>{}, c + 1);
  }
  asm volatile("s_waitcnt vmcnt(0)\n\ts_nop 15\n\ts_nop 15" ::: "memory");
  float v = 0;
#pragma unroll
  for (int q = 0; q < NACC; q++) {
    asm volatile("" : "+a"(acc[q]));
    v += acc[q][0];
  }
  __syncthreads();
  if (sink && v == 1234.5f) sink[0] = v + reinterpret_cast<float*>(lds)[threadIdx.x];
}

int main(int argc, char** argv) {
  const int settle = argc > 1 ? std::atoi(argv[1]) : 1500, timed = argc > 2 ? std::atoi(argv[2]) : 200;
  const int k_bytes = 4096 * 2, nslab = 64, nsets = 5;   // five operand sets: 320 MiB, past the last-level cache
  const size_t bytes = (size_t)4096 * k_bytes;
  char* A[nsets];
  char* B[nsets];
  for (int s = 0; s < nsets; s++) {
    CHECK(hipMalloc(&A[s], bytes));
    CHECK(hipMalloc(&B[s], bytes));
    CHECK(hipMemset(A[s], 1, bytes));
    CHECK(hipMemset(B[s], 2, bytes));
  }
  float* sink;
  CHECK(hipMalloc(&sink, 4));
  hipEvent_t e0, e1;
  CHECK(hipEventCreate(&e0));
  CHECK(hipEventCreate(&e1));
  auto run = [&](auto kern, int threads, const char* name) {
    CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, LDS_BYTES));
    for (int rep = 0; rep < 2; rep++) {
      for (int it = 0; it < settle; it++)   // settle: the clock comes down to where the power limit holds it
        hipLaunchKernelGGL(kern, dim3(256), dim3(threads), LDS_BYTES, 0, A[it % nsets], B[it % nsets], k_bytes, nslab, sink);
      CHECK(hipEventRecord(e0, 0));
      for (int it = 0; it < timed; it++)
        hipLaunchKernelGGL(kern, dim3(256), dim3(threads), LDS_BYTES, 0, A[it % nsets], B[it % nsets], k_bytes, nslab, sink);
      CHECK(hipEventRecord(e1, 0));
      CHECK(hipEventSynchronize(e1));
      float ms;
      CHECK(hipEventElapsedTime(&ms, e0, e1));
      std::printf("%-44s %8.2f us per launch\n", name, ms / timed * 1e3);
    }
  };
  for (int round = 0; round < 2; round++) {
    run(probe_kernel<false, COPY_GLOBAL, 4, false>, 256, "copies alone, global_load_lds_dwordx4");
    run(probe_kernel<false, COPY_BUFFER, 4, false>, 256, "copies alone, buffer_load_dwordx4 lds");
    run(probe_kernel<true, COPY_NONE, 4, false>, 256, "MFMAs alone, four waves");
    run(probe_kernel<true, COPY_GLOBAL, 4, false>, 256, "MFMAs + copies (global), four waves");
    run(probe_kernel<true, COPY_BUFFER, 4, false>, 256, "MFMAs + copies (buffer), four waves");
    run(probe_kernel<true, COPY_GLOBAL, 4, true>, 256, "MFMAs + copies in pairs, four waves");
    run(probe_kernel<true, COPY_NONE, 8, false>, 512, "MFMAs alone, eight waves");
    run(probe_kernel<true, COPY_GLOBAL, 8, false>, 512, "MFMAs + copies (global), eight waves");
  }
  CHECK(hipDeviceSynchronize());
  return 0;
}
