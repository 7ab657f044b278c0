// Measurement aid, not on any product path: what the matrix pipes of this chip sustain when nothing else is in
// the way.  A loop of nothing but matrix instructions on register operands (no LDS, no global memory inside the
// loop), eight wavefronts per compute unit, with the shader clock and the constant 100 MHz clock read around it.
// The encoder GEMMs are rated against the published peak; this loop says how much of that peak the chip delivers
// on operands of a given kind (zeros, random values) at the clock it holds under that load.  Same role as the
// reference's GEMM micro-benchmark (benchmark/turbo_transformers/layers/kernels/matmul_benchmark.cpp:60-70), one
// level further down.
#include "common.h"

namespace ttmi {

typedef float yf4 __attribute__((ext_vector_type(4)));
typedef float yf16 __attribute__((ext_vector_type(16)));
typedef _Float16 yh8 __attribute__((ext_vector_type(8)));
typedef __bf16 yb8 __attribute__((ext_vector_type(8)));

constexpr int kYardThreads = 512;      // eight wavefronts: two per SIMD
constexpr int kYardOperands = 65536;   // elements of the operand pool the registers are filled from

template <typename V>
struct YardMma;
template <>
struct YardMma<yh8> {
  static __device__ __forceinline__ yf4 run16(yh8 a, yh8 b, yf4 c) { return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0); }
  static __device__ __forceinline__ yf16 run32(yh8 a, yh8 b, yf16 c) { return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0); }
};
template <>
struct YardMma<yb8> {
  static __device__ __forceinline__ yf4 run16(yb8 a, yb8 b, yf4 c) { return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0); }
  static __device__ __forceinline__ yf16 run32(yb8 a, yb8 b, yf16 c) { return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0); }
};

// BLOCK = 16: sixteen independent v_mfma_f32_16x16x32 per iteration; BLOCK = 32: eight v_mfma_f32_32x32x16.
// Either way 131072 multiply-adds per wavefront and iteration (16 * 16*16*32 = 8 * 32*32*16).
template <typename E, typename V, int BLOCK>
__global__ __launch_bounds__(kYardThreads) void yardstick_mfma_kernel(int iters, const E* __restrict__ pool, float* sink,
                                                                      unsigned long long* clocks) {
  V a[4], b[4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      a[i][e] = pool[(threadIdx.x * 64 + i * 8 + e) & (kYardOperands - 1)];
      b[i][e] = pool[(threadIdx.x * 64 + 32 + i * 8 + e) & (kYardOperands - 1)];
    }
  float r = 0.f;
  const unsigned long long c0 = __builtin_readcyclecounter(), w0 = wall_clock64();
  if constexpr (BLOCK == 32) {
    yf16 acc[8];
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][e] = 0.f;
    for (int it = 0; it < iters; ++it) {
#pragma unroll
      for (int i = 0; i < 8; ++i) acc[i] = YardMma<V>::run32(a[i & 3], b[(i >> 1) & 3], acc[i]);
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) r += acc[i][0];
  } else {
    yf4 acc[16];
#pragma unroll
    for (int i = 0; i < 16; ++i)
#pragma unroll
      for (int e = 0; e < 4; ++e) acc[i][e] = 0.f;
    for (int it = 0; it < iters; ++it) {
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[i] = YardMma<V>::run16(a[i & 3], b[(i >> 2) & 3], acc[i]);
    }
#pragma unroll
    for (int i = 0; i < 16; ++i) r += acc[i][0];
  }
  const unsigned long long c1 = __builtin_readcyclecounter(), w1 = wall_clock64();
  if (threadIdx.x == 0) {
    clocks[2 * blockIdx.x] = c1 - c0;
    clocks[2 * blockIdx.x + 1] = w1 - w0;
  }
  if (r == 12345.678f) sink[0] = r;  // keeps the accumulators alive; never true for these operands in practice
}

}  // namespace ttmi

using namespace ttmi;

extern "C" int ttmi_yardstick_mfma(int block, int dtype, const void* operands, int iters, int workgroups, float* sink,
                                   uint64_t* clocks, void* stream) {
  TTMI_REQUIRE(block == 16 || block == 32, "block is 16 (16x16x32) or 32 (32x32x16)");
  TTMI_REQUIRE(dtype == TTMI_F16 || dtype == TTMI_BF16, "16-bit element types only");
  TTMI_REQUIRE(operands && sink && clocks && iters > 0 && workgroups > 0 && workgroups <= 65536, "bad argument");
  hipStream_t s = (hipStream_t)stream;
  auto* ck = reinterpret_cast<unsigned long long*>(clocks);
  const dim3 grid((unsigned)workgroups), threads(kYardThreads);
  if (dtype == TTMI_F16) {
    if (block == 16) hipLaunchKernelGGL((yardstick_mfma_kernel<f16, yh8, 16>), grid, threads, 0, s, iters, (const f16*)operands, sink, ck);
    else hipLaunchKernelGGL((yardstick_mfma_kernel<f16, yh8, 32>), grid, threads, 0, s, iters, (const f16*)operands, sink, ck);
  } else {
    if (block == 16) hipLaunchKernelGGL((yardstick_mfma_kernel<bf16, yb8, 16>), grid, threads, 0, s, iters, (const bf16*)operands, sink, ck);
    else hipLaunchKernelGGL((yardstick_mfma_kernel<bf16, yb8, 32>), grid, threads, 0, s, iters, (const bf16*)operands, sink, ck);
  }
  return launch_status("yardstick_mfma_kernel");
}
