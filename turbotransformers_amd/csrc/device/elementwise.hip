// Element-wise and permutation kernels of the encoder layer: AddBiasAct, the head
// split/merge transposes (dense and smart-batch padded forms), embedding lookup, the
// PrepareBertMasks helpers, and small utilities (2-D transpose, dtype convert).
// All are HBM-bound: every thread moves 16-byte vectors, rows are contiguous in lanes.
#include "common.h"

#include <type_traits>

namespace ttmi {

constexpr int kBlock = 256;

// ---------------------------------------------------------------------------- AddBiasAct
// out[m,n] = act(out[m,n] + bias[n])                                  (activation.cpp:33-55)
template <typename T, int VEC, int ACT>
__global__ __launch_bounds__(kBlock) void add_bias_act_kernel(T* __restrict__ out, const T* __restrict__ bias,
                                                              int64_t total_vec, int n_vec) {
  int64_t i = blockIdx.x * (int64_t)kBlock + threadIdx.x;
  const int64_t stride = (int64_t)gridDim.x * kBlock;
  for (; i < total_vec; i += stride) {
    const int c = (int)(i % n_vec) * VEC;
    Vec<T, VEC> o = load_vec<T, VEC>(out + i * VEC);
    Vec<T, VEC> b = load_vec<T, VEC>(bias + c);
#pragma unroll
    for (int j = 0; j < VEC; ++j) o.v[j] = from_float<T>(apply_act<ACT>(to_float(o.v[j]) + to_float(b.v[j])));
    store_vec<T, VEC>(out + i * VEC, o);
  }
}

template <typename T, int ACT>
static int add_bias_act_dispatch(T* out, const T* bias, int64_t m, int64_t n, hipStream_t s) {
  if (m == 0 || n == 0) return 0;
  constexpr int VMAX = 16 / sizeof(T);
  const bool aligned = ((reinterpret_cast<uintptr_t>(out) | reinterpret_cast<uintptr_t>(bias)) & 15) == 0;
  const int64_t total = m * n;
  auto grid_for = [](int64_t nvec) { return (unsigned)std::min<int64_t>(ceil_div(nvec, kBlock), 256 * 32); };
  if (aligned && n % VMAX == 0) {
    hipLaunchKernelGGL((add_bias_act_kernel<T, VMAX, ACT>), dim3(grid_for(total / VMAX)), dim3(kBlock), 0, s,
                       out, bias, total / VMAX, (int)(n / VMAX));
  } else {
    hipLaunchKernelGGL((add_bias_act_kernel<T, 1, ACT>), dim3(grid_for(total)), dim3(kBlock), 0, s, out, bias,
                       total, (int)n);
  }
  return launch_status("add_bias_act");
}

// ------------------------------------------------------------------- head split / merge
// in[T, 3, h, d] + bias[3, h, d] -> q,k,v[B, h, S, d]                (transpose.cpp:347-390)
// One thread per 16-byte chunk of the [T, 3H] input; chunks never straddle a head because
// d % VEC == 0.  PAD form: token t of the packed input belongs to sequence b with
// cu[b] <= t < cu[b+1]; rows s >= len[b] of the outputs are zero-filled (transpose.cpp:501-564).
template <typename T, int VEC, bool PAD>
__global__ __launch_bounds__(kBlock) void split_add_bias_transpose_kernel(
    const T* __restrict__ in, const T* __restrict__ bias, T* __restrict__ q, T* __restrict__ k,
    T* __restrict__ v, const int32_t* __restrict__ cu, int batch, int seq, int heads, int dim) {
  // grid.x = B*S (one output row position per block), threads cover the 3*h*d/VEC chunks.
  const int64_t bs = blockIdx.x;
  const int b = (int)(bs / seq);
  const int s = (int)(bs % seq);
  const int hd = heads * dim;
  int64_t src_row;
  bool valid = true;
  if (PAD) {
    const int start = cu[b];
    const int len = cu[b + 1] - start;
    valid = s < len;
    src_row = (int64_t)start + s;
  } else {
    src_row = bs;
  }
  const int chunks = 3 * hd / VEC;
  for (int c = threadIdx.x; c < chunks; c += kBlock) {
    const int col = c * VEC;           // column inside [3, h, d]
    const int w = col / hd;            // 0:q 1:k 2:v
    const int rem = col - w * hd;
    const int head = rem / dim;
    const int i = rem - head * dim;
    T* dst_base = (w == 0) ? q : (w == 1 ? k : v);
    T* dst = dst_base + (((int64_t)b * heads + head) * seq + s) * dim + i;
    Vec<T, VEC> o;
    if (valid) {
      Vec<T, VEC> x = load_vec<T, VEC>(in + src_row * 3 * hd + col);
      Vec<T, VEC> bb = load_vec<T, VEC>(bias + col);
#pragma unroll
      for (int j = 0; j < VEC; ++j) o.v[j] = from_float<T>(to_float(x.v[j]) + to_float(bb.v[j]));
    } else {
#pragma unroll
      for (int j = 0; j < VEC; ++j) o.v[j] = from_float<T>(0.f);
    }
    store_vec<T, VEC>(dst, o);
  }
}

// in[B, h, S, d] -> out[B, S, h, d]  (dense) or packed out[sum(len), h, d] (PAD)
//                                                     (transpose.cpp:105-156)
template <typename T, int VEC, bool PAD>
__global__ __launch_bounds__(kBlock) void transpose_for_score_kernel(const T* __restrict__ in,
                                                                     T* __restrict__ out,
                                                                     const int32_t* __restrict__ cu, int batch,
                                                                     int seq, int heads, int dim) {
  const int64_t bs = blockIdx.x;
  const int b = (int)(bs / seq);
  const int s = (int)(bs % seq);
  int64_t dst_row = bs;
  if (PAD) {
    const int start = cu[b];
    if (s >= cu[b + 1] - start) return;
    dst_row = (int64_t)start + s;
  }
  const int hd = heads * dim;
  for (int c = threadIdx.x; c < hd / VEC; c += kBlock) {
    const int col = c * VEC;
    const int head = col / dim;
    const int i = col - head * dim;
    Vec<T, VEC> x = load_vec<T, VEC>(in + (((int64_t)b * heads + head) * seq + s) * dim + i);
    store_vec<T, VEC>(out + dst_row * hd + col, x);
  }
}

template <typename T, bool PAD>
static int split_dispatch(const T* in, const T* bias, T* q, T* k, T* v, const int32_t* cu, int64_t batch,
                          int64_t seq, int64_t heads, int64_t dim, hipStream_t s) {
  if (batch * seq == 0) return 0;
  TTMI_REQUIRE(batch * seq < (1ll << 31) && heads * dim * 3 < (1ll << 31), "shape too large");
  constexpr int VMAX = 16 / sizeof(T);
  uintptr_t bits = reinterpret_cast<uintptr_t>(in) | reinterpret_cast<uintptr_t>(bias) |
                   reinterpret_cast<uintptr_t>(q) | reinterpret_cast<uintptr_t>(k) |
                   reinterpret_cast<uintptr_t>(v);
  const dim3 grid((unsigned)(batch * seq));
  if ((bits & 15) == 0 && dim % VMAX == 0) {
    hipLaunchKernelGGL((split_add_bias_transpose_kernel<T, VMAX, PAD>), grid, dim3(kBlock), 0, s, in, bias, q, k,
                       v, cu, (int)batch, (int)seq, (int)heads, (int)dim);
  } else {
    hipLaunchKernelGGL((split_add_bias_transpose_kernel<T, 1, PAD>), grid, dim3(kBlock), 0, s, in, bias, q, k, v,
                       cu, (int)batch, (int)seq, (int)heads, (int)dim);
  }
  return launch_status("split_add_bias_transpose");
}

template <typename T, bool PAD>
static int merge_dispatch(const T* in, T* out, const int32_t* cu, int64_t batch, int64_t seq, int64_t heads,
                          int64_t dim, hipStream_t s) {
  if (batch * seq == 0) return 0;
  TTMI_REQUIRE(batch * seq < (1ll << 31) && heads * dim < (1ll << 31), "shape too large");
  constexpr int VMAX = 16 / sizeof(T);
  uintptr_t bits = reinterpret_cast<uintptr_t>(in) | reinterpret_cast<uintptr_t>(out);
  const dim3 grid((unsigned)(batch * seq));
  if ((bits & 15) == 0 && dim % VMAX == 0) {
    hipLaunchKernelGGL((transpose_for_score_kernel<T, VMAX, PAD>), grid, dim3(kBlock), 0, s, in, out, cu,
                       (int)batch, (int)seq, (int)heads, (int)dim);
  } else {
    hipLaunchKernelGGL((transpose_for_score_kernel<T, 1, PAD>), grid, dim3(kBlock), 0, s, in, out, cu,
                       (int)batch, (int)seq, (int)heads, (int)dim);
  }
  return launch_status("transpose_for_score");
}

// ------------------------------------------------------------------------------ embedding
// out[i,:] (=|+=) table[ids[i],:]                                       (embedding.cpp:49-70)
template <typename T, int VEC, bool ADD>
__global__ __launch_bounds__(kBlock) void lookup_embedding_kernel(T* __restrict__ out,
                                                                  const T* __restrict__ table,
                                                                  const int64_t* __restrict__ ids,
                                                                  int64_t num_ids, int hidden, int64_t vocab,
                                                                  int* __restrict__ err) {
  // one wavefront per id row
  const int64_t row = (int64_t)blockIdx.x * (kBlock / kWave) + threadIdx.x / kWave;
  if (row >= num_ids) return;
  const int64_t id = ids[row];
  T* dst = out + row * hidden;
  if (id < 0 || id >= vocab) {
    // raise the flag the host reads at its next synchronisation, and leave NaN in the row: the buffer may be a
    // recycled block, and whatever it held must not pass for an embedding
    if (threadIdx.x % kWave == 0) *err = 1;
    for (int c = threadIdx.x % kWave; c < hidden; c += kWave) dst[c] = from_float<T>(__builtin_nanf(""));
    return;
  }
  const T* src = table + id * hidden;
  for (int c = (threadIdx.x % kWave) * VEC; c < hidden; c += kWave * VEC) {
    Vec<T, VEC> x = load_vec<T, VEC>(src + c);
    if (ADD) {
      Vec<T, VEC> o = load_vec<T, VEC>(dst + c);
#pragma unroll
      for (int j = 0; j < VEC; ++j) x.v[j] = from_float<T>(to_float(o.v[j]) + to_float(x.v[j]));
    }
    store_vec<T, VEC>(dst + c, x);
  }
}

// Fused BERTEmbedding: e = word[id]; e += type[tt]; e += pos[p]; e = LN(e)
// (bert_embedding.cpp:53-64).  The sums are rounded to the storage type after each add,
// as three separate in-place lookups would; one wavefront per token, row kept in registers.
template <typename T, int VEC, int ITERS>
__global__ __launch_bounds__(kBlock) void bert_embedding_kernel(
    T* __restrict__ out, const int64_t* __restrict__ ids, const int64_t* __restrict__ pos_ids,
    const int64_t* __restrict__ type_ids, const T* __restrict__ word, const T* __restrict__ pos,
    const T* __restrict__ type, const T* __restrict__ gamma, const T* __restrict__ beta, int64_t num_ids,
    int hidden, int64_t vocab, int64_t max_pos, int64_t num_types, float eps, int* __restrict__ err,
    float* __restrict__ out32) {
  const int lane = threadIdx.x % kWave;
  const int64_t row = (int64_t)blockIdx.x * (kBlock / kWave) + threadIdx.x / kWave;
  if (row >= num_ids) return;  // whole wavefront exits together
  const int64_t id = ids[row], p = pos_ids[row], tt = type_ids[row];
  if (id < 0 || id >= vocab || p < 0 || p >= max_pos || tt < 0 || tt >= num_types) {
    // as in lookup_embedding_kernel: flag for the host, NaN in the row
    if (lane == 0) *err = 1;
    for (int c = lane; c < hidden; c += kWave) {
      out[row * hidden + c] = from_float<T>(__builtin_nanf(""));
      if (out32) out32[row * hidden + c] = __builtin_nanf("");
    }
    return;
  }
  const T* wrow = word + id * hidden;
  const T* prow = pos + p * hidden;
  const T* trow = type + tt * hidden;
  float x[ITERS][VEC];
  float sum = 0.f, sumsq = 0.f;
#pragma unroll
  for (int it = 0; it < ITERS; ++it) {
    const int col = (it * kWave + lane) * VEC;
    if (col < hidden) {
      Vec<T, VEC> a = load_vec<T, VEC>(wrow + col);
      Vec<T, VEC> b = load_vec<T, VEC>(trow + col);
      Vec<T, VEC> c = load_vec<T, VEC>(prow + col);
#pragma unroll
      for (int j = 0; j < VEC; ++j) {
        T e = from_float<T>(to_float(a.v[j]) + to_float(b.v[j]));
        e = from_float<T>(to_float(e) + to_float(c.v[j]));
        x[it][j] = to_float(e);
        sum += x[it][j];
        sumsq += x[it][j] * x[it][j];
      }
    } else {
#pragma unroll
      for (int j = 0; j < VEC; ++j) x[it][j] = 0.f;
    }
  }
  sum = group_sum<kWave>(sum);
  sumsq = group_sum<kWave>(sumsq);
  const float mean = sum / (float)hidden;
  const float var = fmaxf(sumsq / (float)hidden - mean * mean, 0.f);  // cancellation on a near-constant row must not go negative
  const float rstd = 1.0f / sqrtf(var + eps);
  T* orow = out + row * hidden;
#pragma unroll
  for (int it = 0; it < ITERS; ++it) {
    const int col = (it * kWave + lane) * VEC;
    if (col < hidden) {
      Vec<T, VEC> g = load_vec<T, VEC>(gamma + col);
      Vec<T, VEC> b = load_vec<T, VEC>(beta + col);
      Vec<T, VEC> o;
#pragma unroll
      for (int j = 0; j < VEC; ++j) {
        const float y = to_float(b.v[j]) + to_float(g.v[j]) * rstd * (x[it][j] - mean);
        o.v[j] = from_float<T>(y);
        if (out32) out32[row * hidden + col + j] = y;
      }
      store_vec<T, VEC>(orow + col, o);
    }
  }
}

// ------------------------------------------------------------------- PrepareBertMasks bits
__global__ void sequence_rows_kernel(int64_t* data, int64_t rows, int64_t cols) {
  int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x;
  const int64_t n = rows * cols, stride = (int64_t)gridDim.x * blockDim.x;
  for (; i < n; i += stride) data[i] = i % cols;
}
__global__ void mask_transform_kernel(const int64_t* src, float* dst, int64_t n) {
  int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (; i < n; i += stride) dst[i] = -10000.0f * (float)(1 - src[i]);  // common.cpp:80
}
__global__ void smart_pad_mask_kernel(float* mask, const int32_t* cu, int64_t batch, int64_t max_seq) {
  int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x;
  const int64_t n = batch * max_seq, stride = (int64_t)gridDim.x * blockDim.x;
  for (; i < n; i += stride) {
    const int64_t b = i / max_seq, t = i % max_seq;
    mask[i] = (t < cu[b + 1] - cu[b]) ? 0.0f : -1e9f;
  }
}

// ------------------------------------------------------------------------------ utilities
// out[c, r] = in[r, c]; 32x32 tiles through LDS (+1 pad), 256 threads = 32 x 8.
template <typename T>
__global__ __launch_bounds__(256) void transpose_2d_kernel(const T* __restrict__ in, T* __restrict__ out,
                                                           int64_t rows, int64_t cols) {
  __shared__ T tile[32][33];
  const int64_t c0 = (int64_t)blockIdx.x * 32, r0 = (int64_t)blockIdx.y * 32;
  const int tx = threadIdx.x % 32, ty = threadIdx.x / 32;
  for (int j = ty; j < 32; j += 8)
    if (r0 + j < rows && c0 + tx < cols) tile[j][tx] = in[(r0 + j) * cols + c0 + tx];
  __syncthreads();
  for (int j = ty; j < 32; j += 8)
    if (c0 + j < cols && r0 + tx < rows) out[(c0 + j) * rows + r0 + tx] = tile[tx][j];
}

// out[o, :] = a[o, :] ++ b[o, :] for `outer` rows; U is the widest unit (16, 4, 2 or 1 bytes) that
// divides both row lengths and all three base addresses.  Lengths are in units of U.
template <typename U>
__global__ __launch_bounds__(256) void concat_kernel(const U* __restrict__ a, const U* __restrict__ b, U* __restrict__ out,
                                                     int64_t outer, int64_t a_len, int64_t b_len) {
  const int64_t row_len = a_len + b_len, total = outer * row_len;
  int64_t i = blockIdx.x * (int64_t)256 + threadIdx.x;
  const int64_t stride = (int64_t)gridDim.x * 256;
  for (; i < total; i += stride) {
    const int64_t o = i / row_len, j = i - o * row_len;
    out[i] = j < a_len ? a[o * a_len + j] : b[o * b_len + (j - a_len)];
  }
}

template <typename S, typename D>
__global__ void convert_kernel(const S* __restrict__ src, D* __restrict__ dst, int64_t n) {
  int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (; i < n; i += stride) dst[i] = from_float<D>(to_float(src[i]));
}

template <typename T>
static int bert_embedding_dispatch(T* out, const int64_t* ids, const int64_t* pos_ids, const int64_t* type_ids,
                                   const T* word, const T* pos, const T* type, const T* gamma, const T* beta,
                                   int64_t num_ids, int64_t hidden, int64_t vocab, int64_t max_pos,
                                   int64_t num_types, float eps, hipStream_t s, float* out32 = nullptr) {
  int* err = async_error_flag();
  TTMI_REQUIRE(err != nullptr, "no async error flag");
  constexpr int VMAX = 16 / sizeof(T);
  uintptr_t bits = reinterpret_cast<uintptr_t>(out) | reinterpret_cast<uintptr_t>(word) |
                   reinterpret_cast<uintptr_t>(pos) | reinterpret_cast<uintptr_t>(type) |
                   reinterpret_cast<uintptr_t>(gamma) | reinterpret_cast<uintptr_t>(beta);
  TTMI_REQUIRE(hidden % VMAX == 0 && (bits & 15) == 0,
               "bert_embedding needs hidden % (16/sizeof(T)) == 0 and 16-byte aligned tensors");
  const int64_t nv = hidden / VMAX;
  TTMI_REQUIRE(nv <= 64 * 8, "hidden too large for the fused embedding kernel");
  const dim3 grid((unsigned)ceil_div(num_ids, kBlock / kWave));
  auto launch = [&](auto iters) {
    constexpr int ITERS = decltype(iters)::value;
    hipLaunchKernelGGL((bert_embedding_kernel<T, VMAX, ITERS>), grid, dim3(kBlock), 0, s, out, ids, pos_ids,
                       type_ids, word, pos, type, gamma, beta, num_ids, (int)hidden, vocab, max_pos, num_types, eps,
                       err, out32);
  };
  if (nv <= 64) launch(std::integral_constant<int, 1>{});
  else if (nv <= 128) launch(std::integral_constant<int, 2>{});
  else if (nv <= 256) launch(std::integral_constant<int, 4>{});
  else launch(std::integral_constant<int, 8>{});
  return launch_status("bert_embedding");
}

// [B,S,H] -> [B,H]; type 0 max, 1 mean, 2 first, 3 last                 (seq_pool.cpp:124-155)
template <typename T>
__global__ void seq_pool_kernel(const T* __restrict__ in, T* __restrict__ out, int64_t batch, int64_t seq,
                                int64_t hidden, int type) {
  const int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x;
  if (i >= batch * hidden) return;
  const int64_t b = i / hidden, c = i % hidden;
  const T* col = in + b * seq * hidden + c;
  float r;
  if (type == 2) {
    r = to_float(col[0]);
  } else if (type == 3) {
    r = to_float(col[(seq - 1) * hidden]);
  } else if (type == 1) {
    r = 0.f;
    for (int64_t s = 0; s < seq; ++s) r += to_float(col[s * hidden]);
    r /= (float)seq;
  } else {
    r = to_float(col[0]);
    for (int64_t s = 1; s < seq; ++s) r = fmaxf(r, to_float(col[s * hidden]));
  }
  out[i] = from_float<T>(r);
}

static unsigned flat_grid(int64_t n) { return (unsigned)std::min<int64_t>(ceil_div(n, 256), 256 * 16); }

}  // namespace ttmi

using namespace ttmi;

extern "C" {

int ttmi_add_bias_act(void* out, const void* bias, int64_t m, int64_t n, int act, int dtype, void* stream) {
  TTMI_REQUIRE(out && bias, "null tensor");
  TTMI_REQUIRE(m >= 0 && n >= 0 && n < (1ll << 31), "bad shape");
  hipStream_t s = (hipStream_t)stream;
  TTMI_DISPATCH_FLOAT(dtype, T, {
    switch (act) {
      case TTMI_ACT_GELU: return (add_bias_act_dispatch<T, TTMI_ACT_GELU>((T*)out, (const T*)bias, m, n, s));
      case TTMI_ACT_TANH: return (add_bias_act_dispatch<T, TTMI_ACT_TANH>((T*)out, (const T*)bias, m, n, s));
      case TTMI_ACT_RELU: return (add_bias_act_dispatch<T, TTMI_ACT_RELU>((T*)out, (const T*)bias, m, n, s));
      default: return fail(TTMI_EINVAL, "unknown activation");
    }
  });
  return 0;
}

int ttmi_split_add_bias_transpose_for_score(const void* in, const void* bias, void* q, void* k, void* v,
                                            int64_t batch, int64_t seq, int64_t heads, int64_t head_dim,
                                            int dtype, void* stream) {
  TTMI_REQUIRE(in && bias && q && k && v, "null tensor");
  TTMI_DISPATCH_FLOAT(dtype, T, return (split_dispatch<T, false>((const T*)in, (const T*)bias, (T*)q, (T*)k,
                                                                  (T*)v, nullptr, batch, seq, heads, head_dim,
                                                                  (hipStream_t)stream)));
  return 0;
}

int ttmi_split_add_bias_transpose_for_score_pad(const void* in, const void* bias, void* q, void* k, void* v,
                                                const int32_t* cu_seqlens, int64_t batch, int64_t max_seq,
                                                int64_t heads, int64_t head_dim, int dtype, void* stream) {
  TTMI_REQUIRE(in && bias && q && k && v && cu_seqlens, "null tensor");
  TTMI_DISPATCH_FLOAT(dtype, T, return (split_dispatch<T, true>((const T*)in, (const T*)bias, (T*)q, (T*)k,
                                                                 (T*)v, cu_seqlens, batch, max_seq, heads,
                                                                 head_dim, (hipStream_t)stream)));
  return 0;
}

int ttmi_transpose_for_score(const void* in, void* out, int64_t batch, int64_t seq, int64_t heads,
                             int64_t head_dim, int dtype, void* stream) {
  TTMI_REQUIRE(in && out, "null tensor");
  TTMI_DISPATCH_FLOAT(dtype, T, return (merge_dispatch<T, false>((const T*)in, (T*)out, nullptr, batch, seq,
                                                                  heads, head_dim, (hipStream_t)stream)));
  return 0;
}

int ttmi_transpose_for_score_pad(const void* in, void* out, const int32_t* cu_seqlens, int64_t batch,
                                 int64_t max_seq, int64_t heads, int64_t head_dim, int dtype, void* stream) {
  TTMI_REQUIRE(in && out && cu_seqlens, "null tensor");
  TTMI_DISPATCH_FLOAT(dtype, T, return (merge_dispatch<T, true>((const T*)in, (T*)out, cu_seqlens, batch,
                                                                 max_seq, heads, head_dim,
                                                                 (hipStream_t)stream)));
  return 0;
}

int ttmi_build_cu_seqlens(const int64_t* host_lens, int64_t batch, int32_t* staging, int32_t* cu_seqlens_dev,
                          void* stream) {
  TTMI_REQUIRE(host_lens && staging && cu_seqlens_dev && batch >= 0, "bad argument");
  int64_t acc = 0;
  staging[0] = 0;
  for (int64_t b = 0; b < batch; ++b) {
    TTMI_REQUIRE(host_lens[b] >= 0, "negative sequence length");
    acc += host_lens[b];
    TTMI_REQUIRE(acc < (1ll << 31), "too many tokens");
    staging[b + 1] = (int32_t)acc;
  }
  TTMI_HIP(hipMemcpyAsync(cu_seqlens_dev, staging, (size_t)(batch + 1) * sizeof(int32_t),
                          hipMemcpyHostToDevice, (hipStream_t)stream));
  return 0;
}

int ttmi_lookup_embedding(void* out, const void* table, const int64_t* ids, int64_t num_ids, int64_t hidden,
                          int64_t vocab, int add, int dtype, void* stream) {
  TTMI_REQUIRE(out && table && ids, "null tensor");
  TTMI_REQUIRE(num_ids >= 0 && hidden >= 0 && hidden < (1ll << 31), "bad shape");
  if (num_ids == 0 || hidden == 0) return 0;
  int* err = async_error_flag();
  TTMI_REQUIRE(err != nullptr, "no async error flag");
  const dim3 grid((unsigned)ceil_div(num_ids, kBlock / kWave));
  hipStream_t s = (hipStream_t)stream;
  TTMI_DISPATCH_FLOAT(dtype, T, {
    constexpr int VMAX = 16 / sizeof(T);
    const bool vec_ok = hidden % VMAX == 0 &&
                        ((reinterpret_cast<uintptr_t>(out) | reinterpret_cast<uintptr_t>(table)) & 15) == 0;
    if (vec_ok) {
      if (add) hipLaunchKernelGGL((lookup_embedding_kernel<T, VMAX, true>), grid, dim3(kBlock), 0, s, (T*)out, (const T*)table, ids, num_ids, (int)hidden, vocab, err);
      else hipLaunchKernelGGL((lookup_embedding_kernel<T, VMAX, false>), grid, dim3(kBlock), 0, s, (T*)out, (const T*)table, ids, num_ids, (int)hidden, vocab, err);
    } else {
      if (add) hipLaunchKernelGGL((lookup_embedding_kernel<T, 1, true>), grid, dim3(kBlock), 0, s, (T*)out, (const T*)table, ids, num_ids, (int)hidden, vocab, err);
      else hipLaunchKernelGGL((lookup_embedding_kernel<T, 1, false>), grid, dim3(kBlock), 0, s, (T*)out, (const T*)table, ids, num_ids, (int)hidden, vocab, err);
    }
  });
  return launch_status("lookup_embedding");
}

int ttmi_bert_embedding(void* out, const int64_t* ids, const int64_t* pos_ids, const int64_t* type_ids,
                        const void* word_table, const void* pos_table, const void* type_table,
                        const void* gamma, const void* beta, int64_t num_ids, int64_t hidden, int64_t vocab,
                        int64_t max_pos, int64_t num_types, float eps, int dtype, void* stream) {
  TTMI_REQUIRE(out && ids && pos_ids && type_ids && word_table && pos_table && type_table && gamma && beta,
               "null tensor");
  if (num_ids == 0) return 0;
  TTMI_DISPATCH_FLOAT(dtype, T, return bert_embedding_dispatch<T>((T*)out, ids, pos_ids, type_ids,
                                                                  (const T*)word_table, (const T*)pos_table,
                                                                  (const T*)type_table, (const T*)gamma,
                                                                  (const T*)beta, num_ids, hidden, vocab, max_pos,
                                                                  num_types, eps, (hipStream_t)stream));
  return 0;
}

int ttmi_bert_embedding_residual32(void* out, float* out_f32, const int64_t* ids, const int64_t* pos_ids,
                                   const int64_t* type_ids, const void* word_table, const void* pos_table,
                                   const void* type_table, const void* gamma, const void* beta, int64_t num_ids,
                                   int64_t hidden, int64_t vocab, int64_t max_pos, int64_t num_types, float eps,
                                   int dtype, void* stream) {
  TTMI_REQUIRE(out && out_f32 && ids && pos_ids && type_ids && word_table && pos_table && type_table && gamma && beta,
               "null tensor");
  if (num_ids == 0) return 0;
  TTMI_DISPATCH_FLOAT(dtype, T, return bert_embedding_dispatch<T>((T*)out, ids, pos_ids, type_ids,
                                                                  (const T*)word_table, (const T*)pos_table,
                                                                  (const T*)type_table, (const T*)gamma,
                                                                  (const T*)beta, num_ids, hidden, vocab, max_pos,
                                                                  num_types, eps, (hipStream_t)stream, out_f32));
  return 0;
}

int ttmi_seq_pool(const void* in, void* out, int64_t batch, int64_t seq, int64_t hidden, int pool_type, int dtype,
                  void* stream) {
  TTMI_REQUIRE(in && out, "null tensor");
  TTMI_REQUIRE(pool_type >= 0 && pool_type <= 3, "unknown pool type");
  TTMI_REQUIRE(seq > 0, "sequence length must be positive");
  if (batch * hidden <= 0) return 0;
  const dim3 grid((unsigned)ceil_div(batch * hidden, 256));
  TTMI_DISPATCH_FLOAT(dtype, T, hipLaunchKernelGGL((seq_pool_kernel<T>), grid, dim3(256), 0, (hipStream_t)stream,
                                                   (const T*)in, (T*)out, batch, seq, hidden, pool_type));
  return launch_status("seq_pool");
}

int ttmi_sequence_rows_i64(int64_t* data, int64_t rows, int64_t cols, void* stream) {
  if (rows * cols <= 0) return 0;
  hipLaunchKernelGGL(sequence_rows_kernel, dim3(flat_grid(rows * cols)), dim3(256), 0, (hipStream_t)stream, data,
                     rows, cols);
  return launch_status("sequence_rows");
}

int ttmi_mask_transform(const int64_t* src, float* dst, int64_t n, void* stream) {
  if (n <= 0) return 0;
  hipLaunchKernelGGL(mask_transform_kernel, dim3(flat_grid(n)), dim3(256), 0, (hipStream_t)stream, src, dst, n);
  return launch_status("mask_transform");
}

int ttmi_smart_pad_mask(float* mask, const int32_t* cu_seqlens, int64_t batch, int64_t max_seq, void* stream) {
  if (batch * max_seq <= 0) return 0;
  hipLaunchKernelGGL(smart_pad_mask_kernel, dim3(flat_grid(batch * max_seq)), dim3(256), 0, (hipStream_t)stream,
                     mask, cu_seqlens, batch, max_seq);
  return launch_status("smart_pad_mask");
}

int ttmi_transpose_2d(const void* in, void* out, int64_t rows, int64_t cols, int dtype, void* stream) {
  TTMI_REQUIRE(in && out, "null tensor");
  if (rows * cols == 0) return 0;
  const dim3 grid((unsigned)ceil_div(cols, 32), (unsigned)ceil_div(rows, 32));
  TTMI_REQUIRE(grid.y < 65536, "too many rows for transpose_2d");
  hipStream_t s = (hipStream_t)stream;
  switch (dtype_size(dtype)) {
    case 4: hipLaunchKernelGGL((transpose_2d_kernel<uint32_t>), grid, dim3(256), 0, s, (const uint32_t*)in, (uint32_t*)out, rows, cols); break;
    case 2: hipLaunchKernelGGL((transpose_2d_kernel<uint16_t>), grid, dim3(256), 0, s, (const uint16_t*)in, (uint16_t*)out, rows, cols); break;
    case 1: hipLaunchKernelGGL((transpose_2d_kernel<uint8_t>), grid, dim3(256), 0, s, (const uint8_t*)in, (uint8_t*)out, rows, cols); break;
    default: return fail(TTMI_EINVAL, "unsupported dtype for transpose_2d");
  }
  return launch_status("transpose_2d");
}

int ttmi_concat(const void* a, const void* b, void* out, int64_t outer, int64_t a_inner, int64_t b_inner, int dtype,
                void* stream) {
  TTMI_REQUIRE(out && (a || a_inner == 0) && (b || b_inner == 0), "null tensor");
  TTMI_REQUIRE(outer >= 0 && a_inner >= 0 && b_inner >= 0, "negative size");
  const int64_t esz = (int64_t)dtype_size(dtype);
  TTMI_REQUIRE(esz > 0, "unsupported dtype for concat");
  if (outer * (a_inner + b_inner) == 0) return 0;
  const int64_t ab = a_inner * esz, bb = b_inner * esz;  // bytes per row
  const uintptr_t bits = reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(b) | reinterpret_cast<uintptr_t>(out) |
                         (uintptr_t)ab | (uintptr_t)bb;
  hipStream_t s = (hipStream_t)stream;
#define TTMI_CONCAT_AS(U)                                                                                             \
  hipLaunchKernelGGL((concat_kernel<U>), dim3(flat_grid(outer * (ab + bb) / (int64_t)sizeof(U))), dim3(256), 0, s,  \
                     (const U*)a, (const U*)b, (U*)out, outer, ab / (int64_t)sizeof(U), bb / (int64_t)sizeof(U))
  if ((bits & 15) == 0) TTMI_CONCAT_AS(uint4);
  else if ((bits & 3) == 0) TTMI_CONCAT_AS(uint32_t);
  else if ((bits & 1) == 0) TTMI_CONCAT_AS(uint16_t);
  else TTMI_CONCAT_AS(uint8_t);
#undef TTMI_CONCAT_AS
  return launch_status("concat");
}

int ttmi_convert(const void* src, int src_dtype, void* dst, int dst_dtype, int64_t n, void* stream) {
  TTMI_REQUIRE(src && dst, "null tensor");
  if (n <= 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  const dim3 grid(flat_grid(n));
  TTMI_DISPATCH_FLOAT(src_dtype, S, {
    TTMI_DISPATCH_FLOAT(dst_dtype, D, {
      hipLaunchKernelGGL((convert_kernel<S, D>), grid, dim3(256), 0, s, (const S*)src, (D*)dst, n);
    });
  });
  return launch_status("convert");
}

}  // extern "C"
