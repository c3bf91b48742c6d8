// A measurement aid, not part of the GEMM path: what the matrix cores of this device deliver on a register-only loop of
// the MFMA instruction the kernels use, under the same power cap, with no memory access at all.  The benchmark reports
// it next to the rate of the headline kernel: the fraction of the nominal peak that is there to be had on the
// benchmark's kind of data (FP16 values spread over [-1, 1)) is below one, because the clock follows the power drawn.
#include "gemmkernels_hip.h"

#include <hip/hip_runtime.h>

#include <type_traits>

#include "gk_internal.hpp"

namespace {

using gk_internal::fail;

typedef _Float16 half8v __attribute__((ext_vector_type(8)));
typedef float float4v __attribute__((ext_vector_type(4)));

constexpr int kProbeWorkgroups = 256 * 4;      // four per CU would fit by threads; registers admit one wave per SIMD
constexpr int kProbeThreads = 256;
constexpr int kFrags = 8;                      // fragments of A and of B per set, as in a 128 x 128 wave tile

template <int I, int N, class F>
__device__ __forceinline__ void unroll(F&& f) {
  if constexpr (I < N) {
    f(std::integral_constant<int, I>{});
    unroll<I + 1, N>(f);
  }
}

// One wave per SIMD: 64 accumulator blocks (all 256 accumulation registers), two sets of eight A and eight B
// fragments that take turns (a K loop brings new fragments every 64 MFMAs), the MFMAs of a set in the serpentine
// order of the GEMM kernels.  Nothing is loaded and nothing is stored.
__global__ void __launch_bounds__(kProbeThreads) mfma_rate_probe_kernel(int iters, int random_operands) {
  const unsigned lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
  half8v a[2][kFrags], b[2][kFrags];
  unsigned s = 0x9E3779B9u * (lane + 64u * wave + 256u * blockIdx.x + 1u);
#pragma unroll
  for (int set = 0; set < 2; ++set)
#pragma unroll
    for (int f = 0; f < kFrags; ++f)
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        s = s * 1664525u + 1013904223u;
        const float u = random_operands ? (float)(s >> 21) * (1.0f / 1024.0f) - 1.0f : 0.0f;      // 2048 values in [-1, 1)
        a[set][f][e] = (_Float16)u;
        s = s * 1664525u + 1013904223u;
        const float v = random_operands ? (float)(s >> 21) * (1.0f / 1024.0f) - 1.0f : 0.0f;
        b[set][f][e] = (_Float16)v;
      }
  // The accumulator block (i, j) lives in the accumulation registers a[4 * (8 * j + i) : + 3], named in the instruction text
  // like the kernels that manage these registers themselves: left to the compiler the loop carried a hundred register
  // moves per pass.  The kernel is given all 256 (the clobber of the highest one says so).
  asm volatile("" ::: "a255");
  auto pass = [&](auto first_c) __attribute__((always_inline)) {
    constexpr bool FIRST = decltype(first_c)::value;
    unroll<0, 2>([&](auto set_c) {
      constexpr int set = decltype(set_c)::value;
      unroll<0, kFrags * kFrags>([&](auto m_c) {
        constexpr int m = decltype(m_c)::value, i = m / kFrags, q = m % kFrags, j = (i & 1) ? kFrags - 1 - q : q;
        constexpr int R = 4 * (kFrags * j + i);
        const half8v va = a[set][i], vb = b[set][j];          // (named here: an operand of an assembly statement does not capture by itself)
        if constexpr (FIRST && set == 0) asm volatile("v_mfma_f32_16x16x32_f16 a[%2:%3], %0, %1, 0" :: "v"(va), "v"(vb), "n"(R), "n"(R + 3));
        else asm volatile("v_mfma_f32_16x16x32_f16 a[%2:%3], %0, %1, a[%2:%3]" :: "v"(va), "v"(vb), "n"(R), "n"(R + 3));
      });
    });
  };
  pass(std::integral_constant<bool, true>{});                  // (the accumulators start from zero)
  for (int it = 1; it < iters; ++it) pass(std::integral_constant<bool, false>{});
  // (the results stay in the registers: nothing is stored)
  asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
}

}  // namespace

extern "C" int gk_probe_matrix_rate(int32_t launches, int32_t iterations, int32_t random_operands, void* stream, double* tflops) {
  if (!tflops) return fail(GK_ERR_INVALID_ARGUMENT, "tflops must not be NULL");
  if (launches < 1 || launches > 100000 || iterations < 1 || iterations > 1000000)
    return fail(GK_ERR_INVALID_ARGUMENT, "launches (1 .. 100000) and iterations (1 .. 1000000) out of range: %d, %d", launches, iterations);
  hipStream_t st = (hipStream_t)stream;
  hipEvent_t e0 = nullptr, e1 = nullptr;
  hipError_t e = hipEventCreate(&e0);
  if (e == hipSuccess) e = hipEventCreate(&e1);
  if (e == hipSuccess) e = hipEventRecord(e0, st);
  for (int l = 0; l < launches && e == hipSuccess; ++l) {
    hipLaunchKernelGGL(mfma_rate_probe_kernel, dim3(kProbeWorkgroups), dim3(kProbeThreads), 0, st, (int)iterations, (int)random_operands);
    e = hipGetLastError();
  }
  if (e == hipSuccess) e = hipEventRecord(e1, st);
  if (e == hipSuccess) e = hipEventSynchronize(e1);
  float ms = 0.0f;
  if (e == hipSuccess) e = hipEventElapsedTime(&ms, e0, e1);
  if (e0) (void)hipEventDestroy(e0);
  if (e1) (void)hipEventDestroy(e1);
  if (e != hipSuccess) return fail(GK_ERR_HIP, "the matrix-core rate probe failed: %s", hipGetErrorString(e));
  // per wave and iteration: 2 sets x 64 MFMAs of 16 x 16 x 32 (2 * 16 * 16 * 32 flop each)
  const double flop = (double)launches * kProbeWorkgroups * (kProbeThreads / 64) * (double)iterations * 2.0 * 64.0 * 16384.0;
  *tflops = ms > 0.0f ? flop / ((double)ms * 1e-3) * 1e-12 : 0.0;
  return GK_OK;
}
