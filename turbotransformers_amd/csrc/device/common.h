// Shared device-side helpers for the gfx950 kernels: element types, 16-byte vector
// access, wave64 reductions and the error plumbing of the C ABI.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <cstdio>
#include <string>

#include "ttmi.h"

namespace ttmi {

constexpr int kWave = 64;  // CDNA wavefront width

using f16 = _Float16;
using bf16 = __bf16;

// ---- error plumbing -------------------------------------------------------------------
void set_error(const std::string& msg);
int fail(int code, const std::string& msg);
int check_hip(hipError_t e, const char* what);

#define TTMI_HIP(expr)                                   \
  do {                                                   \
    int _rc = ::ttmi::check_hip((expr), #expr);          \
    if (_rc != 0) return _rc;                            \
  } while (0)

#define TTMI_REQUIRE(cond, msg)                                            \
  do {                                                                     \
    if (!(cond)) return ::ttmi::fail(TTMI_EINVAL, std::string(msg) + " [" #cond "]"); \
  } while (0)

inline int launch_status(const char* what) { return check_hip(hipGetLastError(), what); }

int* async_error_flag();  // device-visible pinned int, 0 = ok

// ---- kernel-selection switches ----------------------------------------------------------
// Overrides of the launchers' own choices, for A/B timing and for tests of small and ragged shapes.  Each starts
// from an environment variable read ONCE (first use; a launch never scans the environment) and can be changed
// afterwards through ttmi_set_kernel_switch.  kSwitchUnset = the launcher decides.
constexpr int kSwitchUnset = -1;
enum KernelSwitch { kSwitchLargeTile = 0, kSwitchWaveKernel = 1, kSwitchAttentionWaves = 2, kSwitchStaticScratchLimit = 3, kSwitchW4AStages = 4, kSwitchW4SplitK = 5, kNumKernelSwitches = 6 };
int kernel_switch(KernelSwitch which);

// ---- scalar conversion ----------------------------------------------------------------
template <typename T>
__device__ __forceinline__ float to_float(T v) { return static_cast<float>(v); }
template <typename T>
__device__ __forceinline__ T from_float(float v) { return static_cast<T>(v); }

// ---- 16-byte vectors of N elements -----------------------------------------------------
template <typename T, int N>
struct alignas(sizeof(T) * N) Vec {
  T v[N];
};

template <typename T, int N>
__device__ __forceinline__ Vec<T, N> load_vec(const T* p) {
  return *reinterpret_cast<const Vec<T, N>*>(p);
}
template <typename T, int N>
__device__ __forceinline__ void store_vec(T* p, const Vec<T, N>& x) {
  *reinterpret_cast<Vec<T, N>*>(p) = x;
}
// The same store to an address that is only aligned to the element: global memory takes vector stores at any
// alignment (the target's unaligned access mode, which the compiler relies on as well), so this is still one
// instruction; a store that straddles a cache line costs a second request, nothing more.
template <typename T, int N>
struct __attribute__((packed, aligned(alignof(T)))) UnalignedVec {
  Vec<T, N> x;
};
template <typename T, int N>
__device__ __forceinline__ void store_vec_unaligned(T* p, const Vec<T, N>& x) {
  reinterpret_cast<UnalignedVec<T, N>*>(p)->x = x;
}

// ---- wave64 reductions over groups of G lanes (G power of two <= 64) -------------------
template <int G>
__device__ __forceinline__ float group_sum(float v) {
#pragma unroll
  for (int off = G / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, kWave);
  return v;
}
template <int G>
__device__ __forceinline__ float group_max(float v) {
#pragma unroll
  for (int off = G / 2; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, kWave));
  return v;
}

// tanh-form GELU exactly as the reference states it, written through the logistic identity
// 0.5*(1+tanh(u)) == 1/(1+exp(-2u)), u = sqrt(2/pi)*(x + 0.044715 x^3).  With the constants folded
// into one polynomial in x it is 5 VALU operations plus one v_exp_f32 and one v_rcp_f32 (both
// accurate to 1 ulp; a correctly rounded division would cost ten more instructions).
__device__ __forceinline__ float gelu_tanh(float x) {
  constexpr float c1 = -2.0f * 1.4426950408889634f * 0.7978845608028654f;  // exp(-2u) = exp2(x*(c1 + c3 x^2))
  constexpr float c3 = c1 * 0.044715f;
  const float e = __builtin_amdgcn_exp2f(x * __builtin_fmaf(x * x, c3, c1));
  return x * __builtin_amdgcn_rcpf(1.0f + e);
}
__device__ __forceinline__ float fast_tanh(float x) {
  // tanh(x) = 1 - 2/(exp(2x)+1); saturates cleanly at +-1 when exp overflows/underflows
  const float e = __builtin_amdgcn_exp2f(x * (2.0f * 1.4426950408889634f));
  return __builtin_fmaf(-2.0f, __builtin_amdgcn_rcpf(e + 1.0f), 1.0f);
}

template <int ACT>
__device__ __forceinline__ float apply_act(float x) {
  if (ACT == TTMI_ACT_GELU) return gelu_tanh(x);
  if (ACT == TTMI_ACT_TANH) return fast_tanh(x);
  return fmaxf(x, 0.0f);
}

inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

inline size_t dtype_size(int dtype) {
  switch (dtype) {
    case TTMI_F32: return 4;
    case TTMI_F16: return 2;
    case TTMI_BF16: return 2;
    case TTMI_I8: return 1;
    case TTMI_I32: return 4;
    case TTMI_I64: return 8;
    default: return 0;
  }
}

// Dispatch a generic lambda on the floating storage type.
#define TTMI_DISPATCH_FLOAT(dtype, T, ...)                                  \
  switch (dtype) {                                                          \
    case TTMI_F32: { using T = float; __VA_ARGS__; break; }                 \
    case TTMI_F16: { using T = ::ttmi::f16; __VA_ARGS__; break; }           \
    case TTMI_BF16: { using T = ::ttmi::bf16; __VA_ARGS__; break; }         \
    default: return ::ttmi::fail(TTMI_EINVAL, "unsupported dtype");         \
  }

}  // namespace ttmi
