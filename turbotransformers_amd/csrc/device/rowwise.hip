// Row-wise, HBM-bound kernels: LayerNorm / AddBiasLayerNorm and ApplyMaskAndSoftmax.
//
// Layout idea shared by both: a row is owned by a group of G lanes of one wavefront
// (G = 8..64); every lane keeps ITERS 16-byte vectors of the row in registers, so the row
// is read from HBM once and written once, and the two reductions are wave64 shuffles with
// no LDS and no block barrier.  A block is 256 threads = 4 wavefronts = 256/G rows.
// Rows too long for the register budget go to a block-per-row fallback.
#include "common.h"

namespace ttmi {

constexpr int kBlock = 256;

// --------------------------------------------------------------------------- LayerNorm --
// x = out (+ input + bias); mean = sum(x)/n; var = sum(x*x)/n - mean^2;
// out = beta + gamma * (x - mean) * rsqrt(var + eps)      (layer_norm.cpp:144-163)
//
// RES32 = 1: the residual is read from an fp32 copy (`res32`) instead of `input`, and the result is
// also written unrounded to `out32`.  With 16-bit storage this keeps the residual stream of the
// encoder in fp32 -- only GEMM operands are rounded -- at the cost of 12 instead of 6 bytes/element.
// RES32 = 2: in addition the product itself arrives unrounded, in `out32` (which this kernel then overwrites with
// the result, element by element, each by the thread that read it); `out` is only written: 14 bytes/element.
// absmax (optional): TTMI_ABSMAX_SLOTS floats; workgroup b writes max|result| of its rows to slot b and workgroup 0
// zeroes the slots past the grid (the launcher passes it only when the grid fits), so that the dynamic quantisation
// of the next Linear's input finds its scale without a pass of its own.
template <typename T, int VEC, int G, int ITERS, bool ADD, int RES32>
__global__ __launch_bounds__(kBlock) void layer_norm_rows(T* __restrict__ out, const T* __restrict__ input,
                                                          const T* __restrict__ bias,
                                                          const T* __restrict__ gamma,
                                                          const T* __restrict__ beta, int64_t m, int n,
                                                          float eps, const float* res32, float* out32, float* absmax) {
  constexpr int ROWS = kBlock / G;
  const int lane = threadIdx.x % G;
  const int64_t row = (int64_t)blockIdx.x * ROWS + threadIdx.x / G;
  const bool row_ok = row < m;
  T* orow = out + row * n;
  const T* irow = (ADD && !RES32) ? input + row * n : nullptr;

  float x[ITERS][VEC];
  float sum = 0.f, sumsq = 0.f;
#pragma unroll
  for (int it = 0; it < ITERS; ++it) {
    const int col = (it * G + lane) * VEC;
    if (row_ok && col < n) {
      Vec<T, VEC> o;
      if (RES32 != 2) o = load_vec<T, VEC>(orow + col);
      if (ADD && RES32 == 2) {
        Vec<T, VEC> b = load_vec<T, VEC>(bias + col);
#pragma unroll
        for (int j = 0; j < VEC; ++j) x[it][j] = out32[row * n + col + j] + res32[row * n + col + j] + to_float(b.v[j]);
      } else if (ADD && RES32) {
        Vec<T, VEC> b = load_vec<T, VEC>(bias + col);
#pragma unroll
        for (int j = 0; j < VEC; ++j) x[it][j] = to_float(o.v[j]) + res32[row * n + col + j] + to_float(b.v[j]);
      } else if (ADD) {
        Vec<T, VEC> a = load_vec<T, VEC>(irow + col);
        Vec<T, VEC> b = load_vec<T, VEC>(bias + col);
#pragma unroll
        for (int j = 0; j < VEC; ++j) x[it][j] = to_float(o.v[j]) + to_float(a.v[j]) + to_float(b.v[j]);
      } else {
#pragma unroll
        for (int j = 0; j < VEC; ++j) x[it][j] = to_float(o.v[j]);
      }
#pragma unroll
      for (int j = 0; j < VEC; ++j) {
        sum += x[it][j];
        sumsq += x[it][j] * x[it][j];
      }
    } else {
#pragma unroll
      for (int j = 0; j < VEC; ++j) x[it][j] = 0.f;
    }
  }
  sum = group_sum<G>(sum);
  sumsq = group_sum<G>(sumsq);
  const float mean = sum / (float)n;
  const float var = fmaxf(sumsq / (float)n - mean * mean, 0.f);  // cancellation on a near-constant row must not go negative
  const float rstd = 1.0f / sqrtf(var + eps);
  float amax = 0.f;
#pragma unroll
  for (int it = 0; it < ITERS; ++it) {
    const int col = (it * G + lane) * VEC;
    if (row_ok && col < n) {
      Vec<T, VEC> g = load_vec<T, VEC>(gamma + col);
      Vec<T, VEC> b = load_vec<T, VEC>(beta + col);
      Vec<T, VEC> o;
      float y[VEC];
#pragma unroll
      for (int j = 0; j < VEC; ++j) {
        y[j] = to_float(b.v[j]) + to_float(g.v[j]) * rstd * (x[it][j] - mean);
        if (RES32) asm volatile("" : "+v"(y[j]));  // out is the rounding of the fp32 value, not of the exact multiply-add
      }
      // (the stores in loops of their own: an asm statement between two stores keeps them from being merged)
#pragma unroll
      for (int j = 0; j < VEC; ++j) {
        o.v[j] = from_float<T>(y[j]);
        amax = fmaxf(amax, fabsf(to_float(o.v[j])));  // of the value as stored
      }
      if (RES32) {
#pragma unroll
        for (int j = 0; j < VEC; ++j) out32[row * n + col + j] = y[j];
      }
      store_vec<T, VEC>(orow + col, o);
    }
  }
  if (absmax != nullptr) {
    __shared__ float red[kBlock / kWave];
    amax = group_max<kWave>(amax);
    if (threadIdx.x % kWave == 0) red[threadIdx.x / kWave] = amax;
    __syncthreads();
    if (threadIdx.x == 0) {
      float mx = 0.f;
#pragma unroll
      for (int w = 0; w < kBlock / kWave; ++w) mx = fmaxf(mx, red[w]);
      absmax[blockIdx.x] = mx;
    }
    if (blockIdx.x == 0)
      for (int i = (int)gridDim.x + (int)threadIdx.x; i < TTMI_ABSMAX_SLOTS; i += kBlock) absmax[i] = 0.f;
  }
}

// Fallback: one block per row, any n; the row is re-read from L2 for the second pass.
template <typename T, bool ADD, int RES32>
__global__ __launch_bounds__(kBlock) void layer_norm_block(T* __restrict__ out, const T* __restrict__ input,
                                                           const T* __restrict__ bias,
                                                           const T* __restrict__ gamma,
                                                           const T* __restrict__ beta, int64_t m, int n,
                                                           float eps, const float* res32, float* out32) {
  __shared__ float red[2][kBlock / kWave];
  const int64_t row = blockIdx.x;
  T* orow = out + row * n;
  const T* irow = (ADD && !RES32) ? input + row * n : nullptr;
  const float* rrow = RES32 ? res32 + row * n : nullptr;
  float sum = 0.f, sumsq = 0.f;
  for (int c = threadIdx.x; c < n; c += kBlock) {
    float x = RES32 == 2 ? out32[row * n + c] : to_float(orow[c]);
    if (ADD) x = x + (RES32 ? rrow[c] : to_float(irow[c])) + to_float(bias[c]);
    sum += x;
    sumsq += x * x;
  }
  sum = group_sum<kWave>(sum);
  sumsq = group_sum<kWave>(sumsq);
  if (threadIdx.x % kWave == 0) {
    red[0][threadIdx.x / kWave] = sum;
    red[1][threadIdx.x / kWave] = sumsq;
  }
  __syncthreads();
  sum = 0.f;
  sumsq = 0.f;
#pragma unroll
  for (int w = 0; w < kBlock / kWave; ++w) {
    sum += red[0][w];
    sumsq += red[1][w];
  }
  const float mean = sum / (float)n;
  const float var = fmaxf(sumsq / (float)n - mean * mean, 0.f);  // cancellation on a near-constant row must not go negative
  const float rstd = 1.0f / sqrtf(var + eps);
  for (int c = threadIdx.x; c < n; c += kBlock) {
    float x = RES32 == 2 ? out32[row * n + c] : to_float(orow[c]);
    if (ADD) x = x + (RES32 ? rrow[c] : to_float(irow[c])) + to_float(bias[c]);
    float y = to_float(beta[c]) + to_float(gamma[c]) * rstd * (x - mean);
    // the 16-bit output is the rounding of the fp32 one: keep the compiler from folding the conversion into the
    // multiply-add (a mixed-precision fma rounds the exact result once, not the fp32 value)
    if (RES32) asm volatile("" : "+v"(y));
    orow[c] = from_float<T>(y);
    if (RES32) out32[row * n + c] = y;
  }
}

template <typename T, int VEC, int G, int ITERS, bool ADD, int RES32>
static int launch_ln_rows(T* out, const T* input, const T* bias, const T* gamma, const T* beta, int64_t m,
                          int n, float eps, const float* res32, float* out32, hipStream_t s, float* absmax, int* slots_written) {
  constexpr int ROWS = kBlock / G;
  const int64_t grid = ceil_div(m, ROWS);
  if (grid > TTMI_ABSMAX_SLOTS) absmax = nullptr;  // more workgroups than slots: the caller finds the maximum itself
  if (slots_written != nullptr) *slots_written = absmax != nullptr ? TTMI_ABSMAX_SLOTS : 0;
  hipLaunchKernelGGL((layer_norm_rows<T, VEC, G, ITERS, ADD, RES32>), dim3((unsigned)grid), dim3(kBlock), 0, s,
                     out, input, bias, gamma, beta, m, n, eps, res32, out32, absmax);
  return launch_status("layer_norm_rows");
}

template <typename T, bool ADD, int RES32 = 0>
static int layer_norm_dispatch(T* out, const T* input, const T* bias, const T* gamma, const T* beta,
                               int64_t m, int64_t n, float eps, hipStream_t s, const float* res32 = nullptr,
                               float* out32 = nullptr, float* absmax = nullptr, int* slots_written = nullptr) {
  if (slots_written != nullptr) *slots_written = 0;
  if (m == 0 || n == 0) return 0;
  constexpr int VEC = 16 / sizeof(T);
  auto aligned16 = [](const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; };
  const bool vec_ok = (n % VEC == 0) && aligned16(out) && aligned16(gamma) && aligned16(beta) &&
                      (!ADD || ((RES32 || aligned16(input)) && aligned16(bias)));
  if (vec_ok) {
    const int64_t nv = n / VEC;  // 16-byte vectors per row
    // Pick the group width G so that nv = G * ITERS with as little idle lane time as possible.
#define TTMI_LN_CASE(G, ITERS) \
  return launch_ln_rows<T, VEC, G, ITERS, ADD, RES32>(out, input, bias, gamma, beta, m, (int)n, eps, res32, out32, s, absmax, slots_written)
    if (nv <= 16) TTMI_LN_CASE(16, 1);
    if (nv <= 32) TTMI_LN_CASE(32, 1);
    if (nv <= 64) TTMI_LN_CASE(64, 1);
    if (nv <= 96 && nv % 32 == 0) TTMI_LN_CASE(32, 3);  // H=768 fp16/bf16
    if (nv <= 128) TTMI_LN_CASE(64, 2);
    if (nv <= 192) TTMI_LN_CASE(64, 3);                 // H=768 fp32
    if (nv <= 256) TTMI_LN_CASE(64, 4);                 // H=1024 fp32
    if (nv <= 384) TTMI_LN_CASE(64, 6);
    if (nv <= 512) TTMI_LN_CASE(64, 8);
#undef TTMI_LN_CASE
  }
  TTMI_REQUIRE(m < (1ll << 31), "too many rows");
  hipLaunchKernelGGL((layer_norm_block<T, ADD, RES32>), dim3((unsigned)m), dim3(kBlock), 0, s, out, input, bias,
                     gamma, beta, m, (int)n, eps, res32, out32);
  return launch_status("layer_norm_block");
}

// ----------------------------------------------------------------------------- softmax --
// x = score*scale + mask; p = exp(x - max) * (1/sum)        (softmax.cpp:28-81)
// A group of G lanes owns R consecutive rows; all R*ITERS vector loads of score (and mask) are
// issued before the first reduction so that enough bytes are in flight per wavefront.
template <typename T, int VEC, int G, int ITERS, int R, bool MASK_VEC>
__global__ __launch_bounds__(kBlock) void softmax_rows(T* __restrict__ score, const float* __restrict__ mask,
                                                       int64_t rows, int heads, int from_len, int to_len,
                                                       int mask_is_2d, float scale) {
  constexpr int GROUPS = kBlock / G;
  constexpr float kLowest = -3.402823466e+38f;
  const int lane = threadIdx.x % G;
  const int64_t row0 = ((int64_t)blockIdx.x * GROUPS + threadIdx.x / G) * R;
  float x[R][ITERS][VEC];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int64_t row = row0 + r;
    const bool row_ok = row < rows;
    const T* srow = score + row * to_len;
    const float* mrow = nullptr;
    if (mask != nullptr && row_ok) {
      const int64_t b = row / ((int64_t)heads * from_len);
      const int64_t f = row % from_len;
      mrow = mask + (mask_is_2d ? b * to_len : (b * from_len + f) * to_len);
    }
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
      const int col = (it * G + lane) * VEC;
      if (row_ok && col < to_len) {
        const Vec<T, VEC> sv = load_vec<T, VEC>(srow + col);
        if (mrow != nullptr) {
          if (MASK_VEC) {
            const Vec<float, VEC> mv = load_vec<float, VEC>(mrow + col);
#pragma unroll
            for (int j = 0; j < VEC; ++j) x[r][it][j] = to_float(sv.v[j]) * scale + mv.v[j];
          } else {
#pragma unroll
            for (int j = 0; j < VEC; ++j) x[r][it][j] = to_float(sv.v[j]) * scale + mrow[col + j];
          }
        } else {
#pragma unroll
          for (int j = 0; j < VEC; ++j) x[r][it][j] = to_float(sv.v[j]) * scale;
        }
      } else {
#pragma unroll
        for (int j = 0; j < VEC; ++j) x[r][it][j] = kLowest;
      }
    }
  }
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int64_t row = row0 + r;
    const bool row_ok = row < rows;
    float mx = kLowest;
#pragma unroll
    for (int it = 0; it < ITERS; ++it)
#pragma unroll
      for (int j = 0; j < VEC; ++j) mx = fmaxf(mx, x[r][it][j]);
    mx = group_max<G>(mx);
    float sum = 0.f;
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
      const int col = (it * G + lane) * VEC;
#pragma unroll
      for (int j = 0; j < VEC; ++j) {
        const float e = (row_ok && col < to_len) ? __expf(x[r][it][j] - mx) : 0.f;
        x[r][it][j] = e;
        sum += e;
      }
    }
    sum = group_sum<G>(sum);
    const float coef = 1.0f / sum;
    T* srow = score + row * to_len;
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
      const int col = (it * G + lane) * VEC;
      if (row_ok && col < to_len) {
        Vec<T, VEC> o;
#pragma unroll
        for (int j = 0; j < VEC; ++j) o.v[j] = from_float<T>(x[r][it][j] * coef);
        store_vec<T, VEC>(srow + col, o);
      }
    }
  }
}

// Fallback for very long rows: block per row, three passes over L2-resident data.
template <typename T>
__global__ __launch_bounds__(kBlock) void softmax_block(T* __restrict__ score, const float* __restrict__ mask,
                                                        int64_t rows, int heads, int from_len, int to_len,
                                                        int mask_is_2d, float scale) {
  __shared__ float red[kBlock / kWave];
  const int64_t row = blockIdx.x;
  T* srow = score + row * to_len;
  const float* mrow = nullptr;
  if (mask != nullptr) {
    const int64_t b = row / ((int64_t)heads * from_len);
    const int64_t f = row % from_len;
    mrow = mask + (mask_is_2d ? b * to_len : (b * from_len + f) * to_len);
  }
  float mx = -3.402823466e+38f;
  for (int c = threadIdx.x; c < to_len; c += kBlock) {
    float v = to_float(srow[c]) * scale;
    if (mrow) v += mrow[c];
    mx = fmaxf(mx, v);
  }
  mx = group_max<kWave>(mx);
  if (threadIdx.x % kWave == 0) red[threadIdx.x / kWave] = mx;
  __syncthreads();
  mx = red[0];
#pragma unroll
  for (int w = 1; w < kBlock / kWave; ++w) mx = fmaxf(mx, red[w]);
  __syncthreads();
  float sum = 0.f;
  for (int c = threadIdx.x; c < to_len; c += kBlock) {
    float v = to_float(srow[c]) * scale;
    if (mrow) v += mrow[c];
    sum += __expf(v - mx);
  }
  sum = group_sum<kWave>(sum);
  if (threadIdx.x % kWave == 0) red[threadIdx.x / kWave] = sum;
  __syncthreads();
  sum = 0.f;
#pragma unroll
  for (int w = 0; w < kBlock / kWave; ++w) sum += red[w];
  const float coef = 1.0f / sum;
  for (int c = threadIdx.x; c < to_len; c += kBlock) {
    float v = to_float(srow[c]) * scale;
    if (mrow) v += mrow[c];
    srow[c] = from_float<T>(__expf(v - mx) * coef);
  }
}

template <typename T, int VEC, int G, int ITERS>
static int launch_softmax_rows(T* score, const float* mask, int64_t rows, int heads, int from_len, int to_len,
                               int mask_is_2d, float scale, hipStream_t s) {
  constexpr int R = ITERS == 1 ? 4 : (ITERS == 2 ? 2 : 1);
  constexpr int GROUPS = kBlock / G;
  const dim3 grid((unsigned)ceil_div(rows, (int64_t)GROUPS * R));
  // vector loads of the fp32 mask need every mask row to start 4*VEC-byte aligned
  const bool mask_vec = mask != nullptr && (to_len % VEC == 0) &&
                        (reinterpret_cast<uintptr_t>(mask) % (sizeof(float) * VEC) == 0);
  if (mask_vec) {
    hipLaunchKernelGGL((softmax_rows<T, VEC, G, ITERS, R, true>), grid, dim3(kBlock), 0, s, score, mask, rows, heads,
                       from_len, to_len, mask_is_2d, scale);
  } else {
    hipLaunchKernelGGL((softmax_rows<T, VEC, G, ITERS, R, false>), grid, dim3(kBlock), 0, s, score, mask, rows, heads,
                       from_len, to_len, mask_is_2d, scale);
  }
  return launch_status("softmax_rows");
}

template <typename T, int VEC>
static int softmax_vec_dispatch(T* score, const float* mask, int64_t rows, int heads, int from_len, int to_len,
                                int mask_is_2d, float scale, hipStream_t s, bool* done) {
  const int nv = (to_len + VEC - 1) / VEC;
  *done = true;
#define TTMI_SM_CASE(G, ITERS) \
  return launch_softmax_rows<T, VEC, G, ITERS>(score, mask, rows, heads, from_len, to_len, mask_is_2d, scale, s)
  if (nv <= 8) TTMI_SM_CASE(8, 1);
  if (nv <= 16) TTMI_SM_CASE(16, 1);
  if (nv <= 32) TTMI_SM_CASE(32, 1);
  if (nv <= 64) TTMI_SM_CASE(64, 1);
  if (nv <= 128) TTMI_SM_CASE(64, 2);
  if (nv <= 256) TTMI_SM_CASE(64, 4);
  if (nv <= 512) TTMI_SM_CASE(64, 8);
  if (nv <= 1024) TTMI_SM_CASE(64, 16);
#undef TTMI_SM_CASE
  *done = false;
  return 0;
}

template <typename T>
static int softmax_dispatch(T* score, const float* mask, int64_t batch, int64_t heads, int64_t from_len,
                            int64_t to_len, int mask_is_2d, float scale, hipStream_t s) {
  const int64_t rows = batch * heads * from_len;
  if (rows == 0 || to_len == 0) return 0;
  TTMI_REQUIRE(to_len < (1ll << 30) && from_len < (1ll << 30) && heads < (1ll << 30), "dimension too large");
  constexpr int VMAX = 16 / sizeof(T);
  // Row starts are row*to_len elements from a 16-byte aligned base: pick the widest vector
  // that divides to_len so every row start stays aligned for it.
  const bool base_ok = (reinterpret_cast<uintptr_t>(score) & 15) == 0;
  int vec = 1;
  if (base_ok) {
    vec = VMAX;
    while (vec > 1 && (to_len % vec) != 0) vec >>= 1;
  }
  bool done = false;
  int rc = 0;
  switch (vec) {
    case 8: if constexpr (VMAX >= 8) { rc = softmax_vec_dispatch<T, 8>(score, mask, rows, (int)heads, (int)from_len, (int)to_len, mask_is_2d, scale, s, &done); } break;
    case 4: rc = softmax_vec_dispatch<T, 4>(score, mask, rows, (int)heads, (int)from_len, (int)to_len, mask_is_2d, scale, s, &done); break;
    case 2: rc = softmax_vec_dispatch<T, 2>(score, mask, rows, (int)heads, (int)from_len, (int)to_len, mask_is_2d, scale, s, &done); break;
    default: rc = softmax_vec_dispatch<T, 1>(score, mask, rows, (int)heads, (int)from_len, (int)to_len, mask_is_2d, scale, s, &done); break;
  }
  if (done) return rc;
  TTMI_REQUIRE(rows < (1ll << 31), "too many rows");
  hipLaunchKernelGGL((softmax_block<T>), dim3((unsigned)rows), dim3(kBlock), 0, s, score, mask, rows,
                     (int)heads, (int)from_len, (int)to_len, mask_is_2d, scale);
  return launch_status("softmax_block");
}

}  // namespace ttmi

using namespace ttmi;

extern "C" {

int ttmi_layer_norm(void* out, const void* gamma, const void* beta, int64_t m, int64_t n, float eps, int dtype,
                    void* stream) {
  TTMI_REQUIRE(out && gamma && beta, "null tensor");
  TTMI_REQUIRE(m >= 0 && n >= 0 && n < (1ll << 31), "bad shape");
  TTMI_DISPATCH_FLOAT(dtype, T, return (layer_norm_dispatch<T, false>((T*)out, nullptr, nullptr, (const T*)gamma,
                                                                       (const T*)beta, m, n, eps,
                                                                       (hipStream_t)stream)));
  return 0;
}

int ttmi_add_bias_layer_norm(void* out, const void* input, const void* bias, const void* gamma,
                             const void* beta, int64_t m, int64_t n, float eps, int dtype, void* stream) {
  TTMI_REQUIRE(out && input && bias && gamma && beta, "null tensor");
  TTMI_REQUIRE(m >= 0 && n >= 0 && n < (1ll << 31), "bad shape");
  TTMI_DISPATCH_FLOAT(dtype, T, return (layer_norm_dispatch<T, true>((T*)out, (const T*)input, (const T*)bias,
                                                                      (const T*)gamma, (const T*)beta, m, n, eps,
                                                                      (hipStream_t)stream)));
  return 0;
}

int ttmi_add_bias_layer_norm_absmax(void* out, const void* input, const void* bias, const void* gamma, const void* beta,
                                    int64_t m, int64_t n, float eps, int dtype, float* absmax_slots, int* slots_written,
                                    void* stream) {
  TTMI_REQUIRE(out && input && bias && gamma && beta && absmax_slots && slots_written, "null tensor");
  TTMI_REQUIRE(m >= 0 && n >= 0 && n < (1ll << 31), "bad shape");
  TTMI_DISPATCH_FLOAT(dtype, T, return (layer_norm_dispatch<T, true>((T*)out, (const T*)input, (const T*)bias,
                                                                      (const T*)gamma, (const T*)beta, m, n, eps,
                                                                      (hipStream_t)stream, nullptr, nullptr, absmax_slots,
                                                                      slots_written)));
  return 0;
}

int ttmi_add_bias_layer_norm_residual32(void* out, const float* residual_f32, const void* bias, const void* gamma,
                                        const void* beta, float* out_f32, int64_t m, int64_t n, float eps,
                                        int dtype, void* stream) {
  TTMI_REQUIRE(out && residual_f32 && bias && gamma && beta && out_f32, "null tensor");
  TTMI_REQUIRE(m >= 0 && n >= 0 && n < (1ll << 31), "bad shape");
  TTMI_DISPATCH_FLOAT(dtype, T, return (layer_norm_dispatch<T, true, 1>((T*)out, nullptr, (const T*)bias,
                                                                            (const T*)gamma, (const T*)beta, m, n,
                                                                            eps, (hipStream_t)stream, residual_f32,
                                                                            out_f32)));
  return 0;
}

int ttmi_add_bias_layer_norm_product32(void* out, const float* residual_f32, const void* bias, const void* gamma,
                                       const void* beta, float* product_out_f32, int64_t m, int64_t n, float eps,
                                       int dtype, void* stream) {
  TTMI_REQUIRE(out && residual_f32 && bias && gamma && beta && product_out_f32, "null tensor");
  TTMI_REQUIRE(residual_f32 != product_out_f32, "the fp32 product must not alias the residual");
  TTMI_REQUIRE(m >= 0 && n >= 0 && n < (1ll << 31), "bad shape");
  TTMI_DISPATCH_FLOAT(dtype, T, return (layer_norm_dispatch<T, true, 2>((T*)out, nullptr, (const T*)bias,
                                                                         (const T*)gamma, (const T*)beta, m, n, eps,
                                                                         (hipStream_t)stream, residual_f32,
                                                                         product_out_f32)));
  return 0;
}

int ttmi_apply_mask_and_softmax(void* score, const float* mask, int64_t batch, int64_t heads, int64_t from_len,
                                int64_t to_len, int mask_is_2d, float scale, int dtype, void* stream) {
  TTMI_REQUIRE(score != nullptr, "null score");
  TTMI_REQUIRE(batch >= 0 && heads >= 0 && from_len >= 0 && to_len >= 0, "bad shape");
  TTMI_DISPATCH_FLOAT(dtype, T, return softmax_dispatch<T>((T*)score, mask, batch, heads, from_len, to_len,
                                                           mask_is_2d, scale, (hipStream_t)stream));
  return 0;
}

}  // extern "C"
