// Small kernels around the int8 GEMM (dynamic per-tensor activation quantisation and the
// fp32 dequant+bias epilogue) and the per-token row map of a packed (smart) batch.
#include "common.h"

namespace ttmi {

// max|x| in two steps without atomics or a cleared cell: every workgroup of absmax_kernel writes the
// maximum of its share to partial[blockIdx.x]; every workgroup of quantize_kernel then reduces those (at
// most kMaxPartials) values itself before it quantises its share.  Results do not depend on scheduling.
constexpr int kMaxPartials = 512;

__device__ __forceinline__ float block_max_256(float mx, float* red) {
  mx = group_max<kWave>(mx);
  if (threadIdx.x % kWave == 0) red[threadIdx.x / kWave] = mx;
  __syncthreads();
  return fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
}

__global__ __launch_bounds__(256) void absmax_kernel(const float* __restrict__ x, int64_t n, float* __restrict__ partial) {
  __shared__ float red[4];
  float mx = 0.f;
  int64_t i = blockIdx.x * (int64_t)256 + threadIdx.x;
  const int64_t stride = (int64_t)gridDim.x * 256;
  if ((reinterpret_cast<uintptr_t>(x) & 15) == 0) {  // 16-byte loads over the aligned body
    const int64_t n4 = n / 4;
    for (int64_t j = i; j < n4; j += stride) {
      const float4 v = reinterpret_cast<const float4*>(x)[j];
      mx = fmaxf(fmaxf(mx, fmaxf(fabsf(v.x), fabsf(v.y))), fmaxf(fabsf(v.z), fabsf(v.w)));
    }
    i += n4 * 4;
  }
  for (; i < n; i += stride) mx = fmaxf(mx, fabsf(x[i]));
  mx = block_max_256(mx, red);
  if (threadIdx.x == 0) partial[blockIdx.x] = mx;
}

__device__ __forceinline__ int quantize_one(float x, float scale) {
  float r = rintf(x / scale);  // round half to even
  r = fminf(fmaxf(r, -127.f), 127.f);
  return (int)r;
}

// partial: `partials` per-workgroup maxima of |x|, written by absmax_kernel (then scale_dev + 2) or by the kernel
// that produced x.
__global__ __launch_bounds__(256) void quantize_kernel(const float* __restrict__ x, int8_t* __restrict__ q,
                                                       float* __restrict__ scale_dev, const float* __restrict__ partial,
                                                       int partials, int64_t n) {
  __shared__ float red[4];
  float mx = 0.f;
  for (int p = threadIdx.x; p < partials; p += 256) mx = fmaxf(mx, partial[p]);
  mx = block_max_256(mx, red);
  const float scale = mx > 0.f ? mx / 127.0f : 1.0f;
  int64_t i = blockIdx.x * (int64_t)256 + threadIdx.x;
  const int64_t stride = (int64_t)gridDim.x * 256;
  if (i == 0) {
    scale_dev[0] = scale;
    scale_dev[1] = mx;
  }
  if (((reinterpret_cast<uintptr_t>(x) & 15) | (reinterpret_cast<uintptr_t>(q) & 3)) == 0) {  // 4 elements per lane
    const int64_t n4 = n / 4;
    for (int64_t j = i; j < n4; j += stride) {
      const float4 v = reinterpret_cast<const float4*>(x)[j];
      const uint32_t packed = (uint32_t)(quantize_one(v.x, scale) & 255) | ((uint32_t)(quantize_one(v.y, scale) & 255) << 8) |
                              ((uint32_t)(quantize_one(v.z, scale) & 255) << 16) | ((uint32_t)(quantize_one(v.w, scale) & 255) << 24);
      reinterpret_cast<uint32_t*>(q)[j] = packed;
    }
    i += n4 * 4;
  }
  for (; i < n; i += stride) q[i] = (int8_t)quantize_one(x[i], scale);
}

__global__ __launch_bounds__(256) void dequant_bias_kernel(const int32_t* __restrict__ acc,
                                                           const float* __restrict__ act_scale,
                                                           const float* __restrict__ w_scale,
                                                           const float* __restrict__ bias,
                                                           float* __restrict__ out, int64_t total, int n) {
  const float sx = act_scale[0];
  int64_t i = blockIdx.x * (int64_t)256 + threadIdx.x;
  const int64_t stride = (int64_t)gridDim.x * 256;
  for (; i < total; i += stride) {
#pragma clang fp contract(off)  // each product and the sum rounded, as the int8 GEMM's own dequantising store does
    const int c = (int)(i % n);
    float v = (float)acc[i] * sx * w_scale[c];
    if (bias) v = v + bias[c];
    out[i] = v;
  }
}

// Per-output-channel symmetric weight quantisation: one wavefront per row of w[N,K].
__global__ __launch_bounds__(256) void quantize_weight_rows_kernel(const float* __restrict__ w, int8_t* __restrict__ q,
                                                                   float* __restrict__ scales, int64_t n, int64_t k) {
  const int64_t row = (int64_t)blockIdx.x * 4 + threadIdx.x / kWave;
  if (row >= n) return;
  const int lane = threadIdx.x % kWave;
  const float* wr = w + row * k;
  float mx = 0.f;
  for (int64_t c = lane; c < k; c += kWave) mx = fmaxf(mx, fabsf(wr[c]));
  mx = group_max<kWave>(mx);
  const float scale = mx > 0.f ? mx / 127.0f : 1.0f;
  if (lane == 0) scales[row] = scale;
  for (int64_t c = lane; c < k; c += kWave) {
    float r = rintf(wr[c] / scale);
    r = fminf(fmaxf(r, -127.f), 127.f);
    q[row * k + c] = (int8_t)r;
  }
}

__global__ void token_rows_kernel(const int32_t* __restrict__ cu, int batch, int max_seq, int total,
                                  int32_t* __restrict__ rows) {
  const int t = blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= total) return;
  int lo = 0, hi = batch;  // find b with cu[b] <= t < cu[b+1]
  while (hi - lo > 1) {
    const int mid = (lo + hi) >> 1;
    if (cu[mid] <= t) lo = mid; else hi = mid;
  }
  rows[t] = lo * max_seq + (t - cu[lo]);
}

static unsigned flat_grid(int64_t n) { return (unsigned)std::min<int64_t>(ceil_div(n, 256), 256 * 16); }

}  // namespace ttmi

using namespace ttmi;

extern "C" {

int ttmi_quantize_rows_i8(const float* x, int8_t* q, float* scale_dev, int64_t m, int64_t k, void* stream) {
  TTMI_REQUIRE(x && q && scale_dev, "null tensor");
  const int64_t n = m * k;
  if (n <= 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  const int partials = (int)std::max<int64_t>(1, std::min<int64_t>(ceil_div(n, 256 * 16), kMaxPartials));
  static_assert(kMaxPartials + 2 == TTMI_QUANT_SCALE_FLOATS, "scale_dev holds the scale, the maximum and the partial maxima");
  hipLaunchKernelGGL(absmax_kernel, dim3((unsigned)partials), dim3(256), 0, s, x, n, scale_dev + 2);
  const unsigned grid = (unsigned)std::min<int64_t>(ceil_div(n, 256 * 4), 256 * 8);
  hipLaunchKernelGGL(quantize_kernel, dim3(std::max(grid, 1u)), dim3(256), 0, s, x, q, scale_dev, scale_dev + 2, partials, n);
  return launch_status("quantize_rows_i8");
}

int ttmi_quantize_rows_i8_from_absmax(const float* x, int8_t* q, float* scale_dev, const float* absmax_slots, int64_t m,
                                      int64_t k, void* stream) {
  TTMI_REQUIRE(x && q && scale_dev && absmax_slots, "null tensor");
  const int64_t n = m * k;
  if (n <= 0) return 0;
  const unsigned grid = (unsigned)std::min<int64_t>(ceil_div(n, 256 * 4), 256 * 8);
  hipLaunchKernelGGL(quantize_kernel, dim3(std::max(grid, 1u)), dim3(256), 0, (hipStream_t)stream, x, q, scale_dev, absmax_slots,
                     TTMI_ABSMAX_SLOTS, n);
  return launch_status("quantize_rows_i8_from_absmax");
}

int ttmi_quantize_weight_rows_i8(const float* w, int8_t* q, float* scales, int64_t n, int64_t k, void* stream) {
  TTMI_REQUIRE(w && q && scales, "null tensor");
  if (n * k <= 0) return 0;
  hipLaunchKernelGGL(quantize_weight_rows_kernel, dim3((unsigned)ceil_div(n, 4)), dim3(256), 0, (hipStream_t)stream, w, q,
                     scales, n, k);
  return launch_status("quantize_weight_rows_i8");
}

int ttmi_dequant_bias(const int32_t* acc, const float* act_scale_dev, const float* w_scale, const float* bias,
                      float* out, int64_t m, int64_t n, void* stream) {
  TTMI_REQUIRE(acc && act_scale_dev && w_scale && out, "null tensor");
  TTMI_REQUIRE(n < (1ll << 31), "N too large");
  if (m * n <= 0) return 0;
  hipLaunchKernelGGL(dequant_bias_kernel, dim3(flat_grid(m * n)), dim3(256), 0, (hipStream_t)stream, acc,
                     act_scale_dev, w_scale, bias, out, m * n, (int)n);
  return launch_status("dequant_bias");
}

int ttmi_build_token_rows(const int32_t* cu_seqlens, int64_t batch, int64_t max_seq, int64_t total,
                          int32_t* token_rows, void* stream) {
  TTMI_REQUIRE(cu_seqlens && token_rows, "null tensor");
  TTMI_REQUIRE(batch > 0 && batch * max_seq < (1ll << 31) && total < (1ll << 31), "bad shape");
  if (total <= 0) return 0;
  hipLaunchKernelGGL(token_rows_kernel, dim3((unsigned)ceil_div(total, 256)), dim3(256), 0, (hipStream_t)stream,
                     cu_seqlens, (int)batch, (int)max_seq, (int)total, token_rows);
  return launch_status("build_token_rows");
}

}  // extern "C"
