// MFMA GEMM family for gfx950 (CDNA4).
//
//   C[M,N] (+)= A[M,K] * op(B)        A row-major, K contiguous
//   op(B) = B[N,K]^T  ("NK": weights kept K-contiguous, the fast path)
//         | B[K,N]    ("KN": P*V and the generic MatMul)
//
// One kernel template serves fp16, bf16, fp32 and int8: operands move through LDS as
// 16-byte chunks (8 halfs / 4 floats / 16 int8), and one chunk per lane is exactly one
// MFMA operand:
//   fp16/bf16  v_mfma_f32_32x32x16_{f16,bf16}   lane l: row l%32, k = 8*(l/32)..+7
//   int8       v_mfma_i32_32x32x32_i8           lane l: row l%32, k = 16*(l/32)..+15
//   fp32       4 x v_mfma_f32_32x32x2_f32       lane l: row l%32, k = 4*(l/32)+j, j = MFMA index
// (the k order inside a chunk is the same permutation for A and B, so the sum is unchanged).
//
// A workgroup owns a BM x BN tile of C; its WM x WN wavefronts each own a
// (BM/WM) x (BN/WN) sub-tile made of 32x32 MFMA blocks held in fp32/int32 accumulators.
// K advances in steps of 128 bytes per row; LDS is double-buffered (global loads for step
// i+1 are issued into registers before the MFMAs of step i and written to the other stage
// afterwards, one barrier per step).  LDS rows are 128 bytes = 8 chunks, XOR-swizzled by
// row so that the 32 rows an MFMA operand read touches spread over all banks.
//
// Block ids are remapped so that the workgroups resident on one XCD (ids equal mod 8)
// cover neighbouring tiles and share A rows / the weight matrix in that XCD's L2.
#pragma once

#include <map>
#include <mutex>
#include <set>
#include <string>
#include <type_traits>
#include <utility>

#include "common.h"

namespace ttmi {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef int intx16 __attribute__((ext_vector_type(16)));
typedef int intx4 __attribute__((ext_vector_type(4)));
typedef _Float16 halfx8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

// 16 bytes moved as one unit.  may_alias: chunks are views of T-typed memory (global, LDS and
// small per-lane staging arrays), so type-based alias analysis must not reorder them.
struct __attribute__((may_alias)) alignas(16) Chunk {
  uint32_t w[4];
};

template <typename T, int N>
__device__ __forceinline__ Chunk pack_chunk(const T (&tmp)[N]) {
  static_assert(sizeof(T) * N == 16, "a chunk is 16 bytes");
  Chunk c;
  __builtin_memcpy(&c, tmp, 16);
  return c;
}

constexpr int kRowBytes = 128;   // bytes of K per LDS row and per K step
constexpr int kChunks = 8;       // 16-byte chunks per LDS row
constexpr int kNumXcd = 8;
constexpr int kXcdRemapMinTiles = 32;  // below this a problem's tiles are not spread over the XCDs
constexpr int kLdsPerCu = 160 * 1024;

template <typename T>
struct Mma;

template <>
struct Mma<f16> {
  using Acc = floatx16;
  using AccScalar = float;
  static __device__ __forceinline__ void run(const Chunk& a, const Chunk& b, Acc& c) {
    c = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(halfx8, a), __builtin_bit_cast(halfx8, b), c, 0, 0, 0);
  }
};
template <>
struct Mma<bf16> {
  using Acc = floatx16;
  using AccScalar = float;
  static __device__ __forceinline__ void run(const Chunk& a, const Chunk& b, Acc& c) {
    c = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  }
};
template <>
struct Mma<float> {
  using Acc = floatx16;
  using AccScalar = float;
  static __device__ __forceinline__ void run(const Chunk& a, const Chunk& b, Acc& c) {
#pragma unroll
    for (int j = 0; j < 4; ++j)
      c = __builtin_amdgcn_mfma_f32_32x32x2f32(__builtin_bit_cast(float, a.w[j]), __builtin_bit_cast(float, b.w[j]), c, 0, 0, 0);
  }
};
template <>
struct Mma<int8_t> {
  using Acc = intx16;
  using AccScalar = int;
  static __device__ __forceinline__ void run(const Chunk& a, const Chunk& b, Acc& c) {
    c = __builtin_amdgcn_mfma_i32_32x32x32_i8(__builtin_bit_cast(intx4, a), __builtin_bit_cast(intx4, b), c, 0, 0, 0);
  }
};

// Exact unsigned division by a runtime constant (n < 2^31), for row -> (batch, position).
struct FastDiv {
  uint32_t mul = 0, shr = 0, d = 1;
  FastDiv() = default;
  explicit FastDiv(uint32_t denom) : d(denom) {
    if (denom <= 1) { mul = 0; shr = 0; d = 1; return; }
    uint32_t lg = 0;
    while ((1ull << lg) < denom) ++lg;
    const uint32_t p = 31 + lg;
    mul = (uint32_t)(((1ull << p) + denom - 1) / denom);
    shr = p - 32;
  }
  __device__ __forceinline__ uint32_t div(uint32_t n) const { return d == 1 ? n : (__umulhi(n, mul) >> shr); }
};

// Tile index -> (tile row, tile column), walking bands of kBandRows tile rows column by column, so
// that the ~32 workgroups running side by side on one XCD cover a block of about 4 x 8 tiles and
// share 4 A row-panels and 8 B column-panels in that XCD's L2 (row-major order would share one A
// panel and stream 32 different B panels).
constexpr int kBandRows = 4;
__device__ __forceinline__ void tile_coords(int t, int tiles_m, int tiles_n, int& tile_m, int& tile_n) {
  const int band = t / (kBandRows * tiles_n);
  const int idx = t - band * (kBandRows * tiles_n);
  const int rows = min(kBandRows, tiles_m - band * kBandRows);
  tile_n = idx / rows;
  tile_m = band * kBandRows + (idx - tile_n * rows);
}

struct GemmArgs {
  const char* a;
  const char* b;
  int m, n, k;
  int64_t lda, ldb;              // elements
  // batch z -> (z / inner, z % inner); offsets in elements
  int inner;
  int64_t a_outer, a_inner, b_outer, b_inner;
  int tiles_m, tiles_n;
  int k_chunk;  // split-K: blockIdx.y owns K range [y*k_chunk, (y+1)*k_chunk) and z passed to the epilogue is y; 0 = whole K
  // One-wavefront-per-SIMD kernel only: a column at which a new run of tiles starts (0 = none).  Tile columns
  // [0, split_tiles) cover [0, split_col), the last of them ragged; the tiles after them start at split_col again.
  int split_col, split_tiles;
};

// ------------------------------------------------------------------------ epilogues -----
// After the K loop each wavefront transposes its accumulators through LDS so that a lane holds
// 8 consecutive columns of one row; an epilogue then sees (batch z, row m, first column n,
// 8 accumulator values, how many of them are inside the matrix) and writes them with one
// 16-byte store (two for fp32/int32 outputs).  `vec` (set on the host) says whether bases and
// leading dimensions allow 16-byte accesses; otherwise, and on the ragged right edge, the
// epilogue falls back to element stores.
template <typename T>
__device__ __forceinline__ void store_row8(T* p, const float (&v)[8]) {
  if constexpr (sizeof(T) == 2) {
    Vec<T, 8> o;
#pragma unroll
    for (int j = 0; j < 8; ++j) o.v[j] = from_float<T>(v[j]);
    store_vec<T, 8>(p, o);
  } else {
    Vec<T, 4> lo, hi;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      lo.v[j] = from_float<T>(v[j]);
      hi.v[j] = from_float<T>(v[j + 4]);
    }
    store_vec<T, 4>(p, lo);
    store_vec<T, 4>(p + 4, hi);
  }
}

template <typename T>
__device__ __forceinline__ void store_row8_unaligned(T* p, const float (&v)[8]) {  // p aligned to the element only
  if constexpr (sizeof(T) == 2) {
    Vec<T, 8> o;
#pragma unroll
    for (int j = 0; j < 8; ++j) o.v[j] = from_float<T>(v[j]);
    store_vec_unaligned<T, 8>(p, o);
  } else {
    Vec<T, 4> lo, hi;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      lo.v[j] = from_float<T>(v[j]);
      hi.v[j] = from_float<T>(v[j + 4]);
    }
    store_vec_unaligned<T, 4>(p, lo);
    store_vec_unaligned<T, 4>(p + 4, hi);
  }
}

template <typename T>
__device__ __forceinline__ void load_row8(const T* p, float (&v)[8]) {
  if constexpr (sizeof(T) == 2) {
    Vec<T, 8> x = load_vec<T, 8>(p);
#pragma unroll
    for (int j = 0; j < 8; ++j) v[j] = to_float(x.v[j]);
  } else {
    Vec<T, 4> lo = load_vec<T, 4>(p), hi = load_vec<T, 4>(p + 4);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      v[j] = to_float(lo.v[j]);
      v[j + 4] = to_float(hi.v[j]);
    }
  }
}

// The bias of an epilogue (bias_ptr(), may be null) is added by store_tile while the values are
// still in accumulator layout, where a lane owns ONE column per 32x32 block: the kernels fetch
// those few values at the start of a tile, so their latency never shows.
template <int TN, int STRIDE, typename Epi>
__device__ __forceinline__ void load_bias_columns_stride(const Epi& epi, int n_first, int n_limit, float (&bj)[TN]) {
  const auto* bias = epi.bias_ptr();
#pragma unroll
  for (int j = 0; j < TN; ++j) {
    const int n = n_first + j * STRIDE;
    bj[j] = (bias != nullptr && n < n_limit) ? to_float(bias[n]) : 0.f;
  }
}
template <int TN, typename Epi>
__device__ __forceinline__ void load_bias_columns(const Epi& epi, int n_first, int n_limit, float (&bj)[TN]) {
  load_bias_columns_stride<TN, 32>(epi, n_first, n_limit, bj);
}

template <typename T>
struct EpiAlphaBeta {
  using Acc = float;
  T* c;
  int64_t ldc, c_outer, c_inner;
  int inner;
  float alpha, beta;
  bool vec;
  __device__ __forceinline__ const T* bias_ptr() const { return nullptr; }
  // single problem, beta == 0 (what the register-store kernel is launched for)
  __device__ __forceinline__ float finish(float x) const { return x * alpha; }
  __device__ __forceinline__ T* dest8(int m, int n) const { return c + (int64_t)m * ldc + n; }
  __device__ __forceinline__ void store8(int z, int m, int n, float (&v)[8], int valid) const {
    T* p = c + (int64_t)(z / inner) * c_outer + (int64_t)(z % inner) * c_inner + (int64_t)m * ldc + n;
#pragma unroll
    for (int j = 0; j < 8; ++j) v[j] *= alpha;
    if (vec && valid == 8) {
      if (beta != 0.f) {
        float old[8];
        load_row8<T>(p, old);
#pragma unroll
        for (int j = 0; j < 8; ++j) v[j] += beta * old[j];
      }
      store_row8<T>(p, v);
    } else {
      for (int j = 0; j < valid; ++j) {
        float r = v[j];
        if (beta != 0.f) r += beta * to_float(p[j]);
        p[j] = from_float<T>(r);
      }
    }
  }
};

template <typename T, int ACT, bool HAS_ACT, bool HAS_RES>
struct EpiBias {
  using Acc = float;
  T* c;
  const T* bias;
  const T* residual;
  int64_t ldc;
  bool vec;
  __device__ __forceinline__ const T* bias_ptr() const { return bias; }
  __device__ __forceinline__ float finish(float x) const { return HAS_ACT ? apply_act<ACT>(x) : x; }
  __device__ __forceinline__ T* dest8(int m, int n) const { return c + (int64_t)m * ldc + n; }
  __device__ __forceinline__ void store8(int, int m, int n, float (&v)[8], int valid) const {
    const int64_t off = (int64_t)m * ldc + n;
    if (HAS_ACT) {
#pragma unroll
      for (int j = 0; j < 8; ++j) v[j] = apply_act<ACT>(v[j]);
    }
    if (vec && valid == 8) {
      if (HAS_RES) {
        float res[8];
        load_row8<T>(residual + off, res);
#pragma unroll
        for (int j = 0; j < 8; ++j) v[j] += res[j];
      }
      store_row8<T>(c + off, v);
    } else {
      for (int j = 0; j < valid; ++j) {
        float r = v[j];
        if (HAS_RES) r += to_float(residual[off + j]);
        c[off + j] = from_float<T>(r);
      }
    }
  }
};

// acc + bias -> q,k,v[B,h,S,d].  Row m is token (b,s); PAD: packed token -> padded row through
// the per-token map token_rows[m] = b*max_seq + s.  head_dim % 8 == 0 keeps a lane's 8 columns
// inside one head, so they land as one 16-byte store; otherwise elements are placed one by one.
template <typename T, bool PAD>
struct EpiQkvSplit {
  using Acc = float;
  T* q;
  T* k;
  T* v;
  const T* bias;
  const int32_t* token_rows;
  int seq, heads, dim, hidden;
  FastDiv div_seq, div_hidden, div_dim;
  bool vec;
  int v_pitch;  // 0: v is [B,h,S,d]; > 0: v is written transposed, [B,h,d,v_pitch]
  __device__ __forceinline__ const T* bias_ptr() const { return bias; }
  // Columns of the V third are stored by the column pass when V is kept transposed.
  __device__ __forceinline__ bool column_pass() const { return v_pitch > 0; }
  __device__ __forceinline__ int first_column_of_pass() const { return 2 * hidden; }
  // Rows m..m+7 of output column n (n in the V third): eight consecutive sequence positions of
  // one V^T row when they belong to one sequence, one 16-byte store.  A sequence length that is no multiple
  // of 8 shifts the groups of the later sequences off the 16-byte grid: the store is aligned to the element only.
  __device__ __forceinline__ void store_col8(int m, int m_limit, int n, float (&val)[8]) const {
    const uint32_t rem = (uint32_t)(n - 2 * hidden);
    const uint32_t head = div_dim.div(rem);
    const uint32_t i = rem - head * dim;
    const uint32_t prow = PAD ? (uint32_t)token_rows[m] : (uint32_t)m;  // b*seq + s
    const uint32_t b = div_seq.div(prow);
    const uint32_t s = prow - b * seq;
    bool fast = m + 8 <= m_limit && s + 8 <= (uint32_t)seq;
    if (PAD && fast) fast = (uint32_t)token_rows[m + 7] == prow + 7;
    if (fast) {
      store_row8_unaligned<T>(v + (((int64_t)b * heads + head) * dim + i) * v_pitch + s, val);
      return;
    }
    // The group straddles two sequences (or the end of the matrix).  Unrolled with constant indices: a loop with a
    // run-time trip count would index val[] dynamically and push it to scratch memory.
    if (!PAD && seq >= 8) {  // the next sequence starts hidden * v_pitch elements further on
      T* dst = v + (((int64_t)b * heads + head) * dim + i) * v_pitch + s;
      const int64_t hop = vt_hop();
#pragma unroll
      for (int j = 0; j < 8; ++j)
        if (m + j < m_limit) dst[j + (s + j >= (uint32_t)seq ? hop : 0)] = from_float<T>(val[j]);
      return;
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      if (m + j >= m_limit) break;
      const uint32_t pr = PAD ? (uint32_t)token_rows[m + j] : (uint32_t)(m + j);
      const uint32_t bj = div_seq.div(pr);
      v[(((int64_t)bj * heads + head) * dim + i) * v_pitch + (pr - bj * seq)] = from_float<T>(val[j]);
    }
  }
  __device__ __forceinline__ int64_t vt_hop() const { return (int64_t)hidden * v_pitch - seq; }
  __device__ __forceinline__ T* dest(uint32_t b, uint32_t s, uint32_t n) const {
    const uint32_t w = div_hidden.div(n);
    const uint32_t rem = n - w * hidden;
    const uint32_t head = div_dim.div(rem);
    const uint32_t i = rem - head * dim;
    T* base = (w == 0) ? q : (w == 1 ? k : v);
    return base + (((int64_t)b * heads + head) * seq + s) * dim + i;
  }
  // dest(b, s, n) = col_part(n) + row_part(m): the address splits into a part that depends on the column only and an
  // element offset that depends on the row only, so a kernel that stores many rows of few columns (or the reverse)
  // does each division once.
  __device__ __forceinline__ T* col_part(uint32_t n) const {
    const uint32_t w = div_hidden.div(n);
    const uint32_t rem = n - w * hidden;
    const uint32_t head = div_dim.div(rem);
    T* base = (w == 0) ? q : (w == 1 ? k : v);
    return base + (int64_t)head * seq * dim + (rem - head * dim);
  }
  __device__ __forceinline__ int64_t row_part(int m) const {
    const uint32_t prow = PAD ? (uint32_t)token_rows[m] : (uint32_t)m;
    const uint32_t b = div_seq.div(prow);
    return ((int64_t)b * heads * seq + (prow - b * seq)) * dim;
  }
  // Whether `rows` consecutive rows that start at a multiple of `rows` always lie in one sequence, so that
  // row_part(first + r) = row_part(first) + r * dim.
  __device__ __forceinline__ bool rows_share_sequence(int rows) const { return !PAD && seq % rows == 0; }
  // The same split for the transposed V of the column pass: V^T[b, head, i, s] = vt_col_part(n) + vt_row_part(m),
  // m the first of eight consecutive rows; whether the eight are one 16-byte store is vt_rows_contiguous(m, limit).
  __device__ __forceinline__ T* vt_col_part(uint32_t n) const {
    const uint32_t rem = n - 2 * hidden;
    return v + (int64_t)rem * v_pitch;  // (head * dim + i) * v_pitch
  }
  __device__ __forceinline__ int64_t vt_row_part(int m) const {
    const uint32_t prow = PAD ? (uint32_t)token_rows[m] : (uint32_t)m;
    const uint32_t b = div_seq.div(prow);
    return (int64_t)b * hidden * v_pitch + (prow - b * seq);
  }
  __device__ __forceinline__ int64_t vt_row_part(int m, uint32_t& s) const {  // also returns the position in the sequence
    const uint32_t prow = PAD ? (uint32_t)token_rows[m] : (uint32_t)m;
    const uint32_t b = div_seq.div(prow);
    s = prow - b * seq;
    return (int64_t)b * hidden * v_pitch + s;
  }
  __device__ __forceinline__ float finish(float x) const { return x; }
  __device__ __forceinline__ T* dest8(int m, int n) const {  // head_dim % 8 == 0: the eight columns stay in one head
    const uint32_t prow = PAD ? (uint32_t)token_rows[m] : (uint32_t)m;
    const uint32_t b = div_seq.div(prow);
    return dest(b, prow - b * seq, (uint32_t)n);
  }
  __device__ __forceinline__ void store8(int, int m, int n, float (&val)[8], int valid) const {
    if (v_pitch > 0 && n >= 2 * hidden) return;  // left to the column pass (groups of 8 never straddle 2*hidden)
    const uint32_t prow = PAD ? (uint32_t)token_rows[m] : (uint32_t)m;  // b*seq + s
    const uint32_t b = div_seq.div(prow);
    const uint32_t s = prow - b * seq;
    if (vec && valid == 8) {
      store_row8<T>(dest(b, s, (uint32_t)n), val);
    } else {
      for (int j = 0; j < valid; ++j) *dest(b, s, (uint32_t)(n + j)) = from_float<T>(val[j]);
    }
  }
};

struct EpiInt32 {
  using Acc = int;
  int32_t* c;
  int64_t ldc;
  bool vec;
  __device__ __forceinline__ const int32_t* bias_ptr() const { return nullptr; }
  __device__ __forceinline__ void store8(int, int m, int n, int (&v)[8], int valid) const {
    int32_t* p = c + (int64_t)m * ldc + n;
    if (vec && valid == 8) {
      Vec<int32_t, 4> lo, hi;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        lo.v[j] = v[j];
        hi.v[j] = v[j + 4];
      }
      store_vec<int32_t, 4>(p, lo);
      store_vec<int32_t, 4>(p + 4, hi);
    } else {
      for (int j = 0; j < valid; ++j) p[j] = v[j];
    }
  }
};

// int32 accumulators -> fp32: out = float(acc) * act_scale * w_scale[n] (+ bias[n]), the dequantisation
// of the int8 Linear folded into the int8 GEMM.  The operation order is that of the stand-alone
// dequant_bias kernel, so both give the same bits.
struct EpiDequant {
  using Acc = int;
  float* c;
  const float* act_scale;  // device scalar
  const float* w_scale;    // [N]
  const float* bias;       // [N] or null
  int64_t ldc;
  bool vec;
  int act;  // ttmi_act, applied after the bias
  // Optional: kAbsmaxSlots floats that receive max|output| per workgroup (slot = workgroup id, the rest zero), so that
  // the dynamic quantisation of the NEXT Linear's input needs no pass of its own to find its scale.
  float* absmax;
  __device__ __forceinline__ const float* bias_ptr() const { return bias; }
  __device__ __forceinline__ bool has_bias() const { return bias != nullptr; }
  __host__ __device__ __forceinline__ float* absmax_slots() const { return absmax; }
  __device__ __forceinline__ float activate(float x) const {
    if (act == TTMI_ACT_GELU) return apply_act<TTMI_ACT_GELU>(x);
    if (act == TTMI_ACT_TANH) return apply_act<TTMI_ACT_TANH>(x);
    if (act == TTMI_ACT_RELU) return apply_act<TTMI_ACT_RELU>(x);
    return x;
  }
  // v: the bit patterns of the finished values (dequantise() and activate(), applied in accumulator layout)
  __device__ __forceinline__ void store8(int, int m, int n, int (&v)[8], int valid) const {
    float r[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) r[j] = __builtin_bit_cast(float, v[j]);
    float* p = c + (int64_t)m * ldc + n;
    if (vec && valid == 8) {
      store_row8<float>(p, r);
    } else {
      for (int j = 0; j < valid; ++j) p[j] = r[j];
    }
  }
};

// The same dequantisation feeding the head split: q,k,v[B,h,S,d] (fp32) = split(float(acc) * act_scale *
// w_scale[n] + bias[n]), the QKV projection of the quantized attention without the [T,3H] round trip.
// Scaling first, bias second -- the order of dequant_bias followed by SplitAddBiasTransposeForScore.
struct EpiDequantQkvSplit {
  using Acc = int;
  EpiQkvSplit<float, false> split;  // its bias is added here, after the scaling
  const float* act_scale;           // device scalar
  const float* w_scale;             // [N]
  __device__ __forceinline__ const float* bias_ptr() const { return split.bias; }
  __device__ __forceinline__ bool has_bias() const { return true; }
  __host__ __device__ __forceinline__ float* absmax_slots() const { return nullptr; }
  __device__ __forceinline__ float activate(float x) const { return x; }
  __device__ __forceinline__ void store8(int z, int m, int n, int (&v)[8], int valid) const {
    float r[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) r[j] = __builtin_bit_cast(float, v[j]);
    split.store8(z, m, n, r, valid);
  }
};

// The dequantising epilogues scale in ACCUMULATOR layout, where a lane owns one column per 32 x 32 block: the
// activation scale and the lane's few weight scales and biases are fetched once per tile, next to the bias columns
// of the other epilogues (fetched per stored row segment they were 17 dependent loads in front of every store).
// float(acc) * act_scale * w_scale[n], then + bias[n], each product and the sum rounded: the operation order of
// dequant_bias_kernel, so that the fused and the two-kernel form give the same bits.
template <typename Epi>
struct Dequantises : std::false_type {};
template <>
struct Dequantises<EpiDequant> : std::true_type {};
template <>
struct Dequantises<EpiDequantQkvSplit> : std::true_type {};
__device__ __forceinline__ float dequantise(int acc, float act_scale, float w_scale, float bias, bool has_bias) {
#pragma clang fp contract(off)
  float r = (float)acc * act_scale * w_scale;
  if (has_bias) r = r + bias;
  return r;
}
// Slots of the per-workgroup maxima a dequantising GEMM may leave for the quantisation of its consumer.
constexpr int kAbsmaxSlots = 1024;
// End of a workgroup's work: its maximum to its slot; workgroup 0 zeroes the slots no workgroup owns.  `red`: LDS the
// kernel no longer needs (at least 16 floats).  Nothing has to be cleared beforehand and nothing is accumulated
// across launches: every slot is written by every launch.
template <typename Epi>
__device__ __forceinline__ void publish_absmax(const Epi& epi, float lane_max, float* red, int threads) {
  if constexpr (Dequantises<Epi>::value) {
    float* slots = epi.absmax_slots();
    if (slots == nullptr) return;
    __syncthreads();
    lane_max = group_max<kWave>(lane_max);
    if (threadIdx.x % kWave == 0) red[threadIdx.x / kWave] = lane_max;
    __syncthreads();
    if (threadIdx.x == 0) {
      float m = 0.f;
      for (int w = 0; w < threads / kWave; ++w) m = fmaxf(m, red[w]);
      slots[blockIdx.x] = m;
    }
    if (blockIdx.x == 0)
      for (int i = (int)gridDim.x + (int)threadIdx.x; i < kAbsmaxSlots; i += threads) slots[i] = 0.f;
  }
}
// sj[0..TN) = weight scales of the lane's columns, sj[TN] = activation scale; untouched for other epilogues
template <int TN, typename Epi>
__device__ __forceinline__ void load_dequant_columns(const Epi& epi, int n_first, int n_limit, float (&sj)[TN + 1]) {
  if constexpr (Dequantises<Epi>::value) {
    sj[TN] = epi.act_scale[0];
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const int n = n_first + j * 32;
      sj[j] = n < n_limit ? epi.w_scale[n] : 0.f;
    }
  }
}

// -------------------------------------------------------------------------- kernel ------
// LDS rows are 128 bytes and the LDS has 64 four-byte banks (256 bytes per bank cycle): rows r and
// r+2 start on the same bank.  A 128-bit operand read is served 16 lanes (= 16 consecutive tile
// rows, one chunk each) at a time, so the 16 rows must land in 16 different 16-byte slots of the
// 256-byte bank period: slot = (r&1)*8 + physical chunk, with physical chunk = chunk ^ ((r>>1)&7).
__device__ __forceinline__ int swizzle(int row, int chunk) { return chunk ^ ((row >> 1) & 7); }

template <typename Epi>
struct HasColumnPass : std::false_type {};
template <typename T, bool PAD>
struct HasColumnPass<EpiQkvSplit<T, PAD>> : std::true_type {};

// Epilogue shared by the kernels.  acc[i][j][e] is C[row 8*(e/4) + 4*lhalf + e%4][col lrow] of its
// 32x32 block.  Each wavefront stages one 32-row strip of its sub-tile at a time in its own
// slice of LDS (the K-loop buffers are free after the last barrier), then reads it back
// row-major, 8 columns per lane, so that global stores are full 16-byte vectors in 128-byte
// row segments.  An epilogue with a column pass (transposed V of the QKV split) gets the
// columns from first_column_of_pass() on read back column-major instead: 8 rows of one column
// per lane, four adjacent lanes covering 32 consecutive rows = 64 contiguous output bytes.
template <typename T, int TM, int TN, int NT, int LDS_BYTES, typename Epi>
__device__ __forceinline__ void store_tile(typename Mma<T>::Acc (&acc)[TM][TN], const float (&bj)[TN], const float (&sj)[TN + 1],
                                           char* smem, const Epi& epi, const GemmArgs& g, int z, int wave_m0, int wave_n0,
                                           int lane, int wave, float& amax) {
  using AccScalar = typename Mma<T>::AccScalar;
  constexpr int W = TN * 32;             // strip width (columns)
  constexpr int LDW = W + 4;             // padded pitch in words: rows stay 16-byte aligned
  constexpr int LANES_PER_ROW = W / 8;   // lanes sharing one row
  constexpr int PASSES = (32 * LANES_PER_ROW + kWave - 1) / kWave;
  static_assert(NT / kWave * 32 * LDW * 4 <= LDS_BYTES, "epilogue staging exceeds the K-loop LDS");
  const int lrow = lane & 31, lhalf = lane >> 5;
  AccScalar* stage = reinterpret_cast<AccScalar*>(smem) + wave * (32 * LDW);
#pragma unroll
  for (int i = 0; i < TM; ++i) {
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        AccScalar staged;
        if constexpr (Dequantises<Epi>::value) {
          const float r = epi.activate(dequantise(acc[i][j][e], sj[TN], sj[j], bj[j], epi.has_bias()));
          amax = fmaxf(amax, fabsf(r));  // rows past M and columns past N repeat valid rows / are zero: harmless
          staged = __builtin_bit_cast(AccScalar, r);
        } else
          staged = acc[i][j][e] + (AccScalar)bj[j];
        stage[(8 * (e / 4) + 4 * lhalf + (e % 4)) * LDW + j * 32 + lrow] = staged;
      }
    bool row_pass = true;
    if constexpr (HasColumnPass<Epi>::value) {
      if (epi.column_pass()) {
        const int first = epi.first_column_of_pass();
        row_pass = wave_n0 < first;  // wave-uniform
        if (wave_n0 + W > first) {
          constexpr int CPASSES = 4 * W / kWave;
#pragma unroll
          for (int p = 0; p < CPASSES; ++p) {
            const int idx = p * kWave + lane;
            const int rg = idx & 3, c = idx >> 2;
            const int m = wave_m0 + i * 32 + rg * 8, ncol = wave_n0 + c;
            if (m < g.m && ncol < g.n && ncol >= first) {
              AccScalar v[8];
#pragma unroll
              for (int t = 0; t < 8; ++t) v[t] = stage[(rg * 8 + t) * LDW + c];
              epi.store_col8(m, g.m, ncol, v);
            }
          }
        }
      }
    }
#pragma unroll
    for (int p = 0; p < PASSES; ++p) {
      if (!row_pass) break;
      const int idx = p * kWave + lane;          // (row, column group) handled by this lane
      const int r = idx / LANES_PER_ROW, cg = idx % LANES_PER_ROW;
      if (r >= 32) continue;
      const int m = wave_m0 + i * 32 + r;
      const int ncol = wave_n0 + cg * 8;
      const int valid = min(8, g.n - ncol);
      AccScalar v[8];
      const Vec<AccScalar, 4> lo = load_vec<AccScalar, 4>(stage + r * LDW + cg * 8);
      const Vec<AccScalar, 4> hi = load_vec<AccScalar, 4>(stage + r * LDW + cg * 8 + 4);
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        v[t] = lo.v[t];
        v[t + 4] = hi.v[t];
      }
      if (m < g.m && valid > 0) epi.store8(z, m, ncol, v, valid);
    }
  }
}

// DEPTH = number of K steps prefetched into registers ahead of the one being computed (1 or 2).
// Small tiles are latency-bound (one step of MFMA work is shorter than a global load), so the
// 64x64 configuration keeps two steps in flight.
template <typename T, int BM, int BN, int WM, int WN, bool B_KN, bool ALIGNED, int DEPTH, typename Epi>
__global__ __launch_bounds__(WM * WN * kWave) void gemm_kernel(const GemmArgs g, const Epi epi) {
  constexpr int NT = WM * WN * kWave;
  constexpr int KPC = 16 / sizeof(T);          // elements per chunk
  constexpr int BK = kRowBytes / sizeof(T);    // elements of K per step
  constexpr int TM = BM / WM / 32, TN = BN / WN / 32;
  constexpr int A_BYTES = BM * kRowBytes, B_BYTES = BN * kRowBytes, STAGE = A_BYTES + B_BYTES;
  constexpr int A_ITERS = BM * kChunks / NT, B_ITERS = BN * kChunks / NT;
  static_assert(BM * kChunks % NT == 0 && BN * kChunks % NT == 0, "tile/threads mismatch");
  constexpr int KN_CPR = BN * (int)sizeof(T) / 16;  // chunks per k-row of a KN tile
  using Acc = typename Mma<T>::Acc;
  using AccScalar = typename Mma<T>::AccScalar;

  extern __shared__ __align__(16) char smem[];

  // XCD-aware tile order: ids equal mod 8 run on one XCD; give each XCD a contiguous tile range.
  const int tiles = g.tiles_m * g.tiles_n;
  // (with few tiles per problem -- typically many small batched problems -- the grid is one workgroup
  // per tile: padding it to the XCD count would only launch idle workgroups)
  const bool remap = tiles >= kXcdRemapMinTiles;
  const int per_xcd = (tiles + kNumXcd - 1) / kNumXcd;
  const int logical = remap ? (int)(blockIdx.x % kNumXcd) * per_xcd + (int)(blockIdx.x / kNumXcd) : (int)blockIdx.x;
  if (logical >= tiles) {
    if constexpr (Dequantises<Epi>::value)
      if (epi.absmax_slots() != nullptr && threadIdx.x == 0) epi.absmax_slots()[blockIdx.x] = 0.f;  // an idle workgroup still owns a slot
    return;
  }
  int tile_m, tile_n;
  tile_coords(logical, g.tiles_m, g.tiles_n, tile_m, tile_n);
  const int z = blockIdx.z;
  const int m0 = tile_m * BM, n0 = tile_n * BN;

  const T* A = reinterpret_cast<const T*>(g.a) + (int64_t)(z / g.inner) * g.a_outer + (int64_t)(z % g.inner) * g.a_inner;
  const T* B = reinterpret_cast<const T*>(g.b) + (int64_t)(z / g.inner) * g.b_outer + (int64_t)(z % g.inner) * g.b_inner;
  int kdim = g.k, z_epi = z;
  if (g.k_chunk > 0) {  // split-K (NK layout only): this workgroup sums a slice of K into its own partial tile
    const int k_lo = (int)blockIdx.y * g.k_chunk;
    kdim = min(g.k_chunk, g.k - k_lo);
    A += k_lo;
    B += k_lo;
    z_epi = (int)blockIdx.y;
  }

  const int tid = threadIdx.x;
  const int lane = tid % kWave, wave = tid / kWave;
  const int wm0 = (wave / WN) * (BM / WM), wn0 = (wave % WN) * (BN / WN);
  const int lrow = lane & 31, lhalf = lane >> 5;

  Acc acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0;

  Chunk ra[DEPTH][A_ITERS], rb[DEPTH][B_ITERS];

  auto load_chunk = [&](const T* base, int64_t ld, int row, int row_limit, int kcol, int k_limit) -> Chunk {
    // 16 bytes of row `row`, elements kcol..kcol+KPC-1; zero outside [0,row_limit) x [0,k_limit)
    Chunk c{{0u, 0u, 0u, 0u}};
    if (row < row_limit && kcol < k_limit) {
      const T* p = base + (int64_t)row * ld + kcol;
      if (ALIGNED) {
        c = *reinterpret_cast<const Chunk*>(p);
      } else {
        T tmp[KPC];
#pragma unroll
        for (int e = 0; e < KPC; ++e) tmp[e] = (kcol + e < k_limit) ? p[e] : T(0);
        c = pack_chunk(tmp);
      }
    }
    return c;
  };

  auto load_global = [&](int kt, Chunk (&ra)[A_ITERS], Chunk (&rb)[B_ITERS]) {
    const int k0 = kt * BK;
#pragma unroll
    for (int i = 0; i < A_ITERS; ++i) {
      const int c = i * NT + tid;
      ra[i] = load_chunk(A, g.lda, m0 + (c >> 3), g.m, k0 + (c & 7) * KPC, kdim);
    }
#pragma unroll
    for (int i = 0; i < B_ITERS; ++i) {
      const int c = i * NT + tid;
      if (!B_KN) {
        rb[i] = load_chunk(B, g.ldb, n0 + (c >> 3), g.n, k0 + (c & 7) * KPC, kdim);
      } else {
        // B[K,N]: row = k index, columns = n
        rb[i] = load_chunk(B, g.ldb, k0 + c / KN_CPR, kdim, n0 + (c % KN_CPR) * KPC, g.n);
      }
    }
  };

  auto store_lds = [&](int stage, const Chunk (&ra)[A_ITERS], const Chunk (&rb)[B_ITERS]) {
    char* as = smem + stage * STAGE;
    char* bs = as + A_BYTES;
#pragma unroll
    for (int i = 0; i < A_ITERS; ++i) {
      const int c = i * NT + tid;
      const int row = c >> 3;
      *reinterpret_cast<Chunk*>(as + row * kRowBytes + swizzle(row, c & 7) * 16) = ra[i];
    }
#pragma unroll
    for (int i = 0; i < B_ITERS; ++i) {
      const int c = i * NT + tid;
      if (!B_KN) {
        const int row = c >> 3;
        *reinterpret_cast<Chunk*>(bs + row * kRowBytes + swizzle(row, c & 7) * 16) = rb[i];
      } else {
        *reinterpret_cast<Chunk*>(bs + c * 16) = rb[i];  // plain [k][n]
      }
    }
  };

  auto compute = [&](int stage) {
    const char* as = smem + stage * STAGE;
    const char* bs = as + A_BYTES;
#pragma unroll
    for (int kk = 0; kk < kChunks / 2; ++kk) {
      Chunk fa[TM], fb[TN];
      const int ch = 2 * kk + lhalf;
#pragma unroll
      for (int i = 0; i < TM; ++i) {
        const int row = wm0 + i * 32 + lrow;
        fa[i] = *reinterpret_cast<const Chunk*>(as + row * kRowBytes + swizzle(row, ch) * 16);
      }
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        const int col = wn0 + j * 32 + lrow;
        if (!B_KN) {
          fb[j] = *reinterpret_cast<const Chunk*>(bs + col * kRowBytes + swizzle(col, ch) * 16);
        } else {
          const T* bt = reinterpret_cast<const T*>(bs);
          T tmp[KPC];
#pragma unroll
          for (int e = 0; e < KPC; ++e) tmp[e] = bt[(ch * KPC + e) * BN + col];
          fb[j] = pack_chunk(tmp);
        }
      }
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) Mma<T>::run(fa[i], fb[j], acc[i][j]);
    }
  };

  const int ksteps = (kdim + BK - 1) / BK;
  load_global(0, ra[0], rb[0]);
  store_lds(0, ra[0], rb[0]);
  __syncthreads();
  if (DEPTH == 1) {
    for (int kt = 0; kt < ksteps; ++kt) {
      const int cur = kt & 1;
      if (kt + 1 < ksteps) load_global(kt + 1, ra[0], rb[0]);
      compute(cur);
      if (kt + 1 < ksteps) store_lds(cur ^ 1, ra[0], rb[0]);
      __syncthreads();
    }
  } else {
    // register slot s%2 holds K step s+1; loads past the last step return zero chunks without
    // touching memory.  Unrolled by two so that the slot index is a compile-time constant.
    load_global(1, ra[0], rb[0]);
    load_global(2, ra[DEPTH - 1], rb[DEPTH - 1]);
    auto step = [&](int kt, Chunk (&sa)[A_ITERS], Chunk (&sb)[B_ITERS]) {
      const int cur = kt & 1;
      compute(cur);
      store_lds(cur ^ 1, sa, sb);      // step kt+1
      __syncthreads();
      load_global(kt + 3, sa, sb);     // refill the slot just drained
    };
    for (int kt = 0; kt < ksteps; kt += 2) {
      step(kt, ra[0], rb[0]);
      if (kt + 1 < ksteps) step(kt + 1, ra[DEPTH - 1], rb[DEPTH - 1]);
    }
  }

  float bj[TN], sj[TN + 1];
  load_bias_columns<TN>(epi, n0 + wn0 + lrow, g.n, bj);
  load_dequant_columns<TN>(epi, n0 + wn0 + lrow, g.n, sj);
  float amax = 0.f;
  store_tile<T, TM, TN, NT, 2 * STAGE>(acc, bj, sj, smem, epi, g, z_epi, m0 + wm0, n0 + wn0, lane, wave, amax);
  publish_absmax(epi, amax, reinterpret_cast<float*>(smem), NT);
}

// ------------------------------------------------------------------ wavefront kernel -----
// For a handful of rows (one short sequence: M <= 128) the product is a chain of short launches, and what a launch
// costs beyond its fixed 4 us is the bytes its busiest CU has to fetch and the barriers of its K loop.  Here a
// workgroup is ONE wavefront that owns a 32 x 32 tile: its MFMA operand fragments are 16 contiguous bytes of a row
// of A and of W, so every lane fetches its fragments straight from global memory into registers (no LDS, no
// barrier, DEPTH K steps of eight loads in flight), and a 128 x 2304 x 768 product is 288 wavefronts over all CUs
// instead of 72 workgroups over 72.  Tiles walk column by column (the four row tiles of a weight panel are
// neighbours and share it in one XCD's L2).  16-bit types, W as [N,K], K a multiple of the 128-byte step.
template <typename T, int DEPTH, typename Epi>
__global__ __launch_bounds__(kWave) void gemm_wave_kernel(const GemmArgs g, const Epi epi) {
  static_assert(sizeof(T) == 2, "16-bit operands");
  constexpr int BK = kRowBytes / sizeof(T);  // 64 elements per K step, four MFMAs
  using Acc = typename Mma<T>::Acc;
  constexpr int STRIP = 32 * (32 + 4) * 4;   // store_tile's staging strip of one wavefront
  __shared__ __align__(16) char strip[STRIP];

  const int tiles = g.tiles_m * g.tiles_n;
  const bool remap = tiles >= kXcdRemapMinTiles;
  const int per_xcd = (tiles + kNumXcd - 1) / kNumXcd;
  const int logical = remap ? (int)(blockIdx.x % kNumXcd) * per_xcd + (int)(blockIdx.x / kNumXcd) : (int)blockIdx.x;
  if (logical >= tiles) return;
  int tile_m, tile_n;
  tile_coords(logical, g.tiles_m, g.tiles_n, tile_m, tile_n);
  const int m0 = tile_m * 32, n0 = tile_n * 32;
  const int lane = threadIdx.x, lrow = lane & 31, lhalf = lane >> 5;

  int kdim = g.k, k_lo = 0, z_epi = 0;
  if (g.k_chunk > 0) {  // split-K: this wavefront sums a slice of K into its own partial tile
    k_lo = (int)blockIdx.y * g.k_chunk;
    kdim = min(g.k_chunk, g.k - k_lo);
    z_epi = (int)blockIdx.y;
  }
  // rows past the edge are clamped to the last one: their results are never stored
  const T* pa = reinterpret_cast<const T*>(g.a) + (int64_t)min(m0 + lrow, g.m - 1) * g.lda + k_lo + lhalf * 8;
  const T* pb = reinterpret_cast<const T*>(g.b) + (int64_t)min(n0 + lrow, g.n - 1) * g.ldb + k_lo + lhalf * 8;

  float bj[1], sj[2];
  load_bias_columns<1>(epi, n0 + lrow, g.n, bj);
  load_dequant_columns<1>(epi, n0 + lrow, g.n, sj);
  Acc acc[1][1];
#pragma unroll
  for (int e = 0; e < 16; ++e) acc[0][0][e] = 0;

  const int ksteps = kdim / BK;
  Chunk ra[DEPTH][4], rb[DEPTH][4];
  auto fetch = [&](int kt, Chunk (&a)[4], Chunk (&b)[4]) __attribute__((always_inline)) {
    if (kt < ksteps) {
#pragma unroll
      for (int kk = 0; kk < 4; ++kk) {
        a[kk] = *reinterpret_cast<const Chunk*>(pa + kt * BK + kk * 16);
        b[kk] = *reinterpret_cast<const Chunk*>(pb + kt * BK + kk * 16);
      }
    }
  };
#pragma unroll
  for (int d = 0; d < DEPTH; ++d) fetch(d, ra[d], rb[d]);
  for (int kt0 = 0; kt0 < ksteps; kt0 += DEPTH) {
#pragma unroll
    for (int u = 0; u < DEPTH; ++u) {
      if (kt0 + u < ksteps) {
#pragma unroll
        for (int kk = 0; kk < 4; ++kk) Mma<T>::run(ra[u][kk], rb[u][kk], acc[0][0]);
        fetch(kt0 + u + DEPTH, ra[u], rb[u]);
      }
    }
  }
  float amax = 0.f;  // (no dequantising epilogue takes this kernel)
  store_tile<T, 1, 1, kWave, STRIP>(acc, bj, sj, strip, epi, g, z_epi, m0, n0, lane, 0, amax);
}

// ---------------------------------------------------------------------------- split-K -----
// Few output tiles and a long K (one short sequence through the FFN: 24 tiles, 48..96 K steps)
// leave most of the chip idle behind a long serial chain.  Then K is cut into `splits` slices,
// every slice is an ordinary workgroup that stores its fp32 partial tile to a workspace
// [splits][M][N], and a second small kernel sums the slices in a fixed order (so results are
// reproducible) and applies the real epilogue.
struct EpiPartial {
  using Acc = float;
  float* ws;
  int64_t mn;   // M*N
  int64_t ldn;  // N
  bool vec;
  __device__ __forceinline__ const float* bias_ptr() const { return nullptr; }
  __device__ __forceinline__ void store8(int split, int m, int n, float (&v)[8], int valid) const {
    float* p = ws + split * mn + (int64_t)m * ldn + n;
    if (vec && valid == 8) {
      store_row8<float>(p, v);
    } else {
      for (int j = 0; j < valid; ++j) p[j] = v[j];
    }
  }
};

// acc (+ bias) -> an fp32 matrix whatever the operand type: a product that feeds a LayerNorm keeps the precision of
// its accumulators (with bfloat16 storage the rounding of that product to 8 bits is the largest single contribution
// to the deviation of a deep encoder from fp32 arithmetic).
template <typename T>
struct EpiF32 {
  using Acc = float;
  float* c;
  const T* bias;  // may be null
  int64_t ldc;
  bool vec;
  __device__ __forceinline__ const T* bias_ptr() const { return bias; }
  __device__ __forceinline__ float finish(float x) const { return x; }
  __device__ __forceinline__ void store8(int, int m, int n, float (&v)[8], int valid) const {
    float* p = c + (int64_t)m * ldc + n;
    if (vec && valid == 8) {
      store_row8<float>(p, v);
    } else {
      for (int j = 0; j < valid; ++j) p[j] = v[j];
    }
  }
};
template <typename Epi>
struct StoresF32 : std::false_type {};
template <typename T>
struct StoresF32<EpiF32<T>> : std::true_type {};

template <typename Epi>
__global__ __launch_bounds__(256) void splitk_reduce_kernel(const float* __restrict__ ws, int splits, int m, int n, bool vec,
                                                            const Epi epi) {
  const int groups = (n + 7) / 8;
  const int64_t idx = blockIdx.x * (int64_t)256 + threadIdx.x;
  const int row = (int)(idx / groups), ncol = (int)(idx % groups) * 8;
  if (row >= m) return;
  const int valid = min(8, n - ncol);
  float v[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) v[j] = 0.f;
  for (int sidx = 0; sidx < splits; ++sidx) {
    const float* p = ws + ((int64_t)sidx * m + row) * n + ncol;
    if (vec && valid == 8) {
      float x[8];
      load_row8<float>(p, x);
#pragma unroll
      for (int j = 0; j < 8; ++j) v[j] += x[j];
    } else {
      for (int j = 0; j < valid; ++j) v[j] += p[j];
    }
  }
  const auto* bias = epi.bias_ptr();
  if (bias != nullptr)
    for (int j = 0; j < valid; ++j) v[j] += to_float(bias[ncol + j]);
  epi.store8(0, row, ncol, v, valid);
}

// The reduction of a split-K GEMM that feeds AddBiasLayerNorm, with the normalisation folded in:
// one workgroup per output row sums the slices (fixed order), adds bias and residual, keeps the row in
// registers (ITERS float4 per thread), and writes LN(x) -- one launch and one pass over the row
// instead of a reduce kernel, a 16-bit round trip and a LayerNorm kernel.  Needs n % 4 == 0,
// n <= 1024 * ITERS and rows of every operand aligned to four elements.   mean / variance as in layer_norm.cpp:144-163 of the reference.
template <typename T, int ITERS>
__global__ __launch_bounds__(256) void splitk_reduce_layer_norm_kernel(const float* __restrict__ ws, int splits, int m, int n,
                                                                      const T* __restrict__ bias, const T* residual,
                                                                      const float* residual32, const T* __restrict__ gamma,
                                                                      const T* __restrict__ beta, T* out, float* out32, float eps) {
  __shared__ float red[2][4];
  const int row = blockIdx.x;
  const int64_t mn = (int64_t)m * n;
  float x[ITERS][4];
  float sum = 0.f, sumsq = 0.f;
#pragma unroll
  for (int it = 0; it < ITERS; ++it) {
    const int col = (it * 256 + threadIdx.x) * 4;
#pragma unroll
    for (int j = 0; j < 4; ++j) x[it][j] = 0.f;
    if (col < n) {
      const float* p = ws + (int64_t)row * n + col;
      for (int sidx = 0; sidx < splits; ++sidx) {
        const float4 v = *reinterpret_cast<const float4*>(p + sidx * mn);
        x[it][0] += v.x; x[it][1] += v.y; x[it][2] += v.z; x[it][3] += v.w;
      }
      const Vec<T, 4> b = load_vec<T, 4>(bias + col);
      float r[4];
      if (residual32 != nullptr) {
        const float4 v = *reinterpret_cast<const float4*>(residual32 + (int64_t)row * n + col);
        r[0] = v.x; r[1] = v.y; r[2] = v.z; r[3] = v.w;
      } else {
        const Vec<T, 4> v = load_vec<T, 4>(residual + (int64_t)row * n + col);
#pragma unroll
        for (int j = 0; j < 4; ++j) r[j] = to_float(v.v[j]);
      }
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        x[it][j] += to_float(b.v[j]) + r[j];
        sum += x[it][j];
        sumsq += x[it][j] * x[it][j];
      }
    }
  }
  sum = group_sum<kWave>(sum);
  sumsq = group_sum<kWave>(sumsq);
  if (threadIdx.x % kWave == 0) {
    red[0][threadIdx.x / kWave] = sum;
    red[1][threadIdx.x / kWave] = sumsq;
  }
  __syncthreads();
  sum = red[0][0] + red[0][1] + red[0][2] + red[0][3];
  sumsq = red[1][0] + red[1][1] + red[1][2] + red[1][3];
  const float mean = sum / (float)n;
  const float var = fmaxf(sumsq / (float)n - mean * mean, 0.f);  // cancellation on a near-constant row must not go negative
  const float rstd = 1.0f / sqrtf(var + eps);
#pragma unroll
  for (int it = 0; it < ITERS; ++it) {
    const int col = (it * 256 + threadIdx.x) * 4;
    if (col < n) {
      const Vec<T, 4> gm = load_vec<T, 4>(gamma + col), bt = load_vec<T, 4>(beta + col);
      Vec<T, 4> o;
      float y[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        y[j] = to_float(bt.v[j]) + to_float(gm.v[j]) * rstd * (x[it][j] - mean);
        o.v[j] = from_float<T>(y[j]);
      }
      store_vec<T, 4>(out + (int64_t)row * n + col, o);
      if (out32 != nullptr) *reinterpret_cast<float4*>(out32 + (int64_t)row * n + col) = make_float4(y[0], y[1], y[2], y[3]);
    }
  }
}

// ------------------------------------------------------------------ fast-path kernel -----
// Same tiling, for the shapes the encoder actually runs (B given as [N,K], 16-byte aligned
// operands, K a multiple of the 128-byte K step).  Two differences from the general kernel:
//   * global -> LDS copies are `global_load_lds_dwordx4` DMA loads: a wavefront instruction
//     moves 8 tile rows (64 lanes x 16 bytes) straight into LDS, no VGPR staging, no
//     ds_write.  The LDS side is linear in the lane id, so the XOR swizzle is applied on the
//     global side: lane l fills physical chunk l%8 of row l/8 and therefore fetches logical
//     chunk (l%8) ^ ((row>>1)&7) of that row.  Rows past the M / N edge are clamped to the
//     last valid row (their results are never stored).
//   * MFMA operand fragments are double-buffered in registers: the LDS reads of k-substep
//     kk+1 are issued before the MFMAs of kk.
//   * the K loop runs over a ring of NS stages, NS - 1 K steps in flight while one is multiplied: two for the
//     256-row tiles (a step is 0.5-1.3 us of matrix work), four for the 128 x 64 tile.
// LDS bytes of the fast kernel: NS K-loop stages, or one stage plus the epilogue staging area
// (which starts at the second stage and may run past the last), whichever is larger.
template <int BM, int BN, int WM, int WN>
constexpr int fast_epilogue_bytes() { return WM * WN * 32 * (BN / WN + 4) * 4; }
template <int BM, int BN, int WM, int WN, int NS = 2>
constexpr int fast_lds_bytes() {
  constexpr int stage = (BM + BN) * kRowBytes;
  constexpr int rest = (NS - 1) * stage;
  return stage + (fast_epilogue_bytes<BM, BN, WM, WN>() > rest ? fast_epilogue_bytes<BM, BN, WM, WN>() : rest);
}

// Barrier that publishes DMA-filled LDS: every wavefront first waits for its own global->LDS loads
// (vmcnt counts them; nothing obliges the compiler to place that wait in front of the barrier), then the
// workgroup synchronises, so that afterwards any wavefront may read rows fetched by any other.
__device__ __forceinline__ void dma_landed_barrier() {
  __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0), other counters untouched
  __syncthreads();
}
// The same with the N youngest vector memory operations of the wavefront allowed to stay in flight (they complete
// in order, so everything older has landed).  Written as instructions: __syncthreads() is a fence as well, and in
// front of a fence the compiler waits for EVERY outstanding vector memory operation, the DMA loads of the later
// stages included.  The wavefront's own LDS reads are waited for, so that the stage it has read may be refilled.
template <int N>
__device__ __forceinline__ void dma_landed_barrier_but() {
  static_assert(N >= 0 && N < 64, "vmcnt is a six-bit counter");
  asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" : : "n"(N) : "memory");
}

template <typename T, int BM, int BN, int WM, int WN, int NS, typename Epi>
__global__ __launch_bounds__(WM * WN * kWave) void gemm_fast_kernel(const GemmArgs g, const Epi epi) {
  static_assert(NS >= 2 && NS <= 4, "stages of the K-loop ring");
  constexpr int NW = WM * WN, NT = NW * kWave;
  constexpr int KPC = 16 / sizeof(T);
  constexpr int BK = kRowBytes / sizeof(T);
  constexpr int TM = BM / WM / 32, TN = BN / WN / 32;
  constexpr int A_BYTES = BM * kRowBytes, B_BYTES = BN * kRowBytes, STAGE = A_BYTES + B_BYTES;
  constexpr int A_LOADS = BM / 8 / NW, B_LOADS = BN / 8 / NW;  // DMA instructions per wave and K step
  static_assert(BM / 8 % NW == 0 && BN / 8 % NW == 0, "tile rows must split evenly over the wavefronts");
  using Acc = typename Mma<T>::Acc;
  typedef __attribute__((address_space(3))) char lds_char;

  extern __shared__ __align__(16) char smem[];

  // Persistent workgroups: the grid holds at most as many workgroups as stay resident and each
  // walks over several tiles.  XCD x owns the contiguous tile range [x*per_xcd, (x+1)*per_xcd);
  // its workgroups (ids equal to x mod 8) stride through it together.  Between two tiles the
  // first K step of the next tile is fetched (DMA into stage 0) before the epilogue of the
  // finished tile runs out of the other half of LDS.
  const int tiles = g.tiles_m * g.tiles_n;
  // With fewer than kXcdRemapMinTiles tiles per problem the grid is simply one workgroup per tile.
  const bool remap = tiles >= kXcdRemapMinTiles;
  const int per_xcd = (tiles + kNumXcd - 1) / kNumXcd;
  const int xcd = (int)(blockIdx.x % kNumXcd), stride = remap ? (int)(gridDim.x / kNumXcd) : (int)gridDim.x;
  const int xcd_end = remap ? min((xcd + 1) * per_xcd, tiles) : tiles;
  int logical = remap ? xcd * per_xcd + (int)(blockIdx.x / kNumXcd) : (int)blockIdx.x;
  if (logical >= xcd_end) {
    if constexpr (Dequantises<Epi>::value)
      if (epi.absmax_slots() != nullptr && threadIdx.x == 0) epi.absmax_slots()[blockIdx.x] = 0.f;  // an idle workgroup still owns a slot
    return;
  }
  const int z = blockIdx.z;
  const T* A = reinterpret_cast<const T*>(g.a) + (int64_t)(z / g.inner) * g.a_outer + (int64_t)(z % g.inner) * g.a_inner;
  const T* B = reinterpret_cast<const T*>(g.b) + (int64_t)(z / g.inner) * g.b_outer + (int64_t)(z % g.inner) * g.b_inner;

  const int tid = threadIdx.x;
  const int lane = tid % kWave, wave = tid / kWave;
  const int wm0 = (wave / WN) * (BM / WM), wn0 = (wave % WN) * (BN / WN);
  const int lrow = lane & 31, lhalf = lane >> 5;
  lds_char* lds0 = reinterpret_cast<lds_char*>(reinterpret_cast<uintptr_t>(smem));
  // byte offsets of this lane's operand rows inside a stage (swizzle folded in per k-substep)
  const int a_row0 = (wm0 + lrow) * kRowBytes, b_row0 = A_BYTES + (wn0 + lrow) * kRowBytes;
  const int swz = ((lrow >> 1) & 7);  // rows wm0 + 32 i + lrow share (row>>1)&7 with lrow
  int ksteps = g.k / BK, z_epi = z;
  if (g.k_chunk > 0) {  // split-K: this workgroup multiplies one K slice into its own partial tile
    const int k_lo = (int)blockIdx.y * g.k_chunk;
    ksteps = min(g.k_chunk, g.k - k_lo) / BK;
    A += k_lo;
    B += k_lo;
    z_epi = (int)blockIdx.y;
  }

  // per-lane source pointers of the DMA loads (advanced by one K step per issue)
  const T* pa[A_LOADS];
  const T* pb[B_LOADS];
  auto point_at = [&](int tile) {
    int tile_m, tile_n;
    tile_coords(tile, g.tiles_m, g.tiles_n, tile_m, tile_n);
    const int m0 = tile_m * BM, n0 = tile_n * BN;
    const int sub = lane >> 3, p = lane & 7;
#pragma unroll
    for (int i = 0; i < A_LOADS; ++i) {
      const int row = (wave * A_LOADS + i) * 8 + sub;
      const int c = p ^ ((row >> 1) & 7);
      pa[i] = A + (int64_t)min(m0 + row, g.m - 1) * g.lda + c * KPC;
    }
#pragma unroll
    for (int i = 0; i < B_LOADS; ++i) {
      const int row = (wave * B_LOADS + i) * 8 + sub;
      const int c = p ^ ((row >> 1) & 7);
      pb[i] = B + (int64_t)min(n0 + row, g.n - 1) * g.ldb + c * KPC;
    }
  };

  // The DMA builtin exists only in the device pass; the host pass of this translation unit
  // needs the kernel body just to emit the launch stub.
#if defined(__HIP_DEVICE_COMPILE__)
  auto issue = [&](int stage) {
    lds_char* as = lds0 + stage * STAGE + wave * (A_LOADS * 1024);
    lds_char* bs = lds0 + stage * STAGE + A_BYTES + wave * (B_LOADS * 1024);
#pragma unroll
    for (int i = 0; i < A_LOADS; ++i) {
      __builtin_amdgcn_global_load_lds(pa[i], as + i * 1024, 16, 0, 0);
      pa[i] += BK;
    }
#pragma unroll
    for (int i = 0; i < B_LOADS; ++i) {
      __builtin_amdgcn_global_load_lds(pb[i], bs + i * 1024, 16, 0, 0);
      pb[i] += BK;
    }
  };
#else
  auto issue = [&](int) { (void)lds0; };
#endif

  auto read_frags = [&](const char* st, int kk, Chunk (&fa)[TM], Chunk (&fb)[TN]) {
    const int off = ((2 * kk + lhalf) ^ swz) << 4;
#pragma unroll
    for (int i = 0; i < TM; ++i) fa[i] = *reinterpret_cast<const Chunk*>(st + a_row0 + i * 32 * kRowBytes + off);
#pragma unroll
    for (int j = 0; j < TN; ++j) fb[j] = *reinterpret_cast<const Chunk*>(st + b_row0 + j * 32 * kRowBytes + off);
  };

  // Software pipeline of one K step (4 k-substeps kk, TM*TN MFMAs each):
  //   kk = 0,1,2 : LDS reads of substep kk+1 interleaved with the MFMAs of kk
  //   wait for the DMA of the next stage + barrier   (everyone has also read all of this stage)
  //   issue the DMA of step kt+NS into the stage just drained
  //   kk = 3     : LDS reads of substep 0 of the NEXT stage interleaved with the MFMAs of kk = 3
  // so neither the LDS latency nor the barrier leaves the MFMA pipe without queued work.
  // sched_group_barrier pins the interleaving (mask 0x100 = LDS read, 0x008 = MFMA).
  constexpr int READS = TM + TN, MMAS = TM * TN;
  Acc acc[TM][TN];
  auto mma_step = [&](Chunk (&fa)[TM], Chunk (&fb)[TN]) {
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j) Mma<T>::run(fa[i], fb[j], acc[i][j]);
  };
  auto interleave = [&]() {
    // MFMA first: its operands were read one substep ago, so the wait in front of it does not
    // cover the reads issued after it.
    constexpr int MF = (sizeof(T) == 4) ? 4 * MMAS : MMAS;  // fp32: 4 MFMA instructions per Mma::run
    constexpr int PER = (MF - 1) / READS;
    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
#pragma unroll
    for (int r = 0; r < READS; ++r) {
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x008, PER, 0);
    }
    __builtin_amdgcn_sched_group_barrier(0x008, MF - 1 - PER * READS, 0);
  };

  point_at(logical);
  issue(0);
  float amax = 0.f;  // max |output| of this workgroup's tiles (dequantising epilogues)
  for (;;) {
    int tile_m, tile_n;
    tile_coords(logical, g.tiles_m, g.tiles_n, tile_m, tile_n);
    const int m0 = tile_m * BM, n0 = tile_n * BN;
    float bj[TN], sj[TN + 1];
    load_bias_columns<TN>(epi, n0 + wn0 + lrow, g.n, bj);
    load_dequant_columns<TN>(epi, n0 + wn0 + lrow, g.n, sj);
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[i][j][e] = 0;

    dma_landed_barrier();  // step 0 has landed; the previous tile's staging area has been read out
#pragma unroll
    for (int st = 1; st < NS; ++st)
      if (st < ksteps) issue(st);
    Chunk fa[2][TM], fb[2][TN];
    read_frags(smem, 0, fa[0], fb[0]);
    int cur = 0;
    for (int kt = 0; kt < ksteps; ++kt) {
      const int nxt = cur + 1 == NS ? 0 : cur + 1;
      const char* st = smem + cur * STAGE;
      const char* st_next = smem + nxt * STAGE;
      read_frags(st, 1, fa[1], fb[1]);
      mma_step(fa[0], fb[0]);
      interleave();
      read_frags(st, 2, fa[0], fb[0]);
      mma_step(fa[1], fb[1]);
      interleave();
      read_frags(st, 3, fa[1], fb[1]);
      mma_step(fa[0], fb[0]);
      interleave();
      // step kt+1 is complete, and everyone has read all of this stage.  Steps kt+2 .. kt+NS-1 (those that
      // exist) stay in flight: each is the youngest A_LOADS + B_LOADS operations of this wavefront.
      if constexpr (NS == 2) {
        dma_landed_barrier();
      } else {
        constexpr int LPS = A_LOADS + B_LOADS;
        const int younger = min(kt + NS - 1, ksteps - 1) - (kt + 1);
        if (NS >= 4 && younger >= 2) dma_landed_barrier_but<(NS >= 4 ? 2 : 0) * LPS>();
        else if (younger >= 1) dma_landed_barrier_but<LPS>();
        else dma_landed_barrier_but<0>();
      }
      if (kt + NS < ksteps) issue(cur);
      read_frags(st_next, 0, fa[0], fb[0]);  // harmless on the last step
      mma_step(fa[1], fb[1]);
      interleave();
      cur = nxt;
    }
    __syncthreads();  // all LDS reads of this tile are done

    const int next = logical + stride;
    if (next < xcd_end) {  // stage 0 is free: fetch the next tile's first K step
      point_at(next);
      issue(0);
      // Let it land before the epilogue starts.  With an LDS DMA in flight the compiler puts a vmcnt(0) in
      // front of every staging read of the epilogue, which would also wait for the previous strip's global
      // stores, one round trip per strip; after this wait the strips' stores are issued back to back.
      __builtin_amdgcn_s_waitcnt(0x0F70);
    }
    store_tile<T, TM, TN, NT, fast_lds_bytes<BM, BN, WM, WN, NS>() - STAGE>(acc, bj, sj, smem + STAGE, epi, g, z_epi, m0 + wm0,
                                                                             n0 + wn0, lane, wave, amax);
    if (next >= xcd_end) break;
    logical = next;
  }
  publish_absmax(epi, amax, reinterpret_cast<float*>(smem), NT);
}

// ------------------------------------------------------------------------ launching -----
// Dry run: while a thread has a string installed here, the launchers below write the name of the kernel variant
// they would launch (tile, wavefronts, K split) into it and launch nothing.  ttmi_gemm_describe uses it, so the
// answer comes from the very code path that picks the kernel.
static thread_local std::string* tl_describe = nullptr;
static bool describe_only(const char* family, int waves, int bm, int bn, int splits = 1) {
  if (tl_describe == nullptr) return false;
  *tl_describe = std::string(family) + std::to_string(waves) + "w_" + std::to_string(bm) + "x" + std::to_string(bn);
  if (splits > 1) *tl_describe += "_splitk" + std::to_string(splits);
  return true;
}

// A dequantising epilogue that was asked for per-workgroup maxima gets them only from a launch whose workgroups fit
// the slots; otherwise the request is dropped and the caller told (tl_absmax_written stays 0), and it finds the
// maximum with a pass of its own.
static thread_local int tl_absmax_written = 0;
template <typename Epi>
static bool absmax_grid_ok(const Epi& epi, unsigned grid_x, int batch) {
  if constexpr (Dequantises<Epi>::value) {
    if (epi.absmax_slots() == nullptr) return true;
    if (grid_x > (unsigned)kAbsmaxSlots || batch != 1) return false;
    tl_absmax_written = kAbsmaxSlots;
  }
  return true;
}
template <typename Epi>
static Epi without_absmax(Epi epi) {
  if constexpr (std::is_same<Epi, EpiDequant>::value) epi.absmax = nullptr;
  return epi;
}

// Kernels that use more than 64 KB of dynamic LDS need the limit raised once per kernel and device.
static int allow_large_lds(const void* kern, int bytes) {
  static std::mutex mu;
  static std::set<std::pair<const void*, int>> done;
  int dev = 0;
  TTMI_HIP(hipGetDevice(&dev));
  std::lock_guard<std::mutex> lock(mu);
  if (done.count({kern, dev}) != 0) return 0;
  TTMI_HIP(hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, bytes));
  done.insert({kern, dev});
  return 0;
}

template <typename T, int BM, int BN, int WM, int WN, bool B_KN, bool ALIGNED, typename Epi>
static int launch_config(GemmArgs g, const Epi& epi, int batch, hipStream_t s) {
  constexpr int NT = WM * WN * kWave;
  constexpr int LDS = 2 * (BM + BN) * kRowBytes;
  if (describe_only("reg", WM * WN, BM, BN)) return 0;
  g.tiles_m = (g.m + BM - 1) / BM;
  g.tiles_n = (g.n + BN - 1) / BN;
  const int64_t tiles = (int64_t)g.tiles_m * g.tiles_n;
  TTMI_REQUIRE(tiles < (1ll << 30) && batch < 65536, "GEMM grid too large");
  const unsigned grid_x = tiles >= kXcdRemapMinTiles ? (unsigned)(ceil_div(tiles, kNumXcd) * kNumXcd) : (unsigned)tiles;
  constexpr int DEPTH = (BM * BN <= 64 * 64 && ALIGNED) ? 2 : 1;
  if (!absmax_grid_ok(epi, grid_x, batch)) return launch_config<T, BM, BN, WM, WN, B_KN, ALIGNED>(g, without_absmax(epi), batch, s);
  auto kern = gemm_kernel<T, BM, BN, WM, WN, B_KN, ALIGNED, DEPTH, Epi>;
  if (LDS > 64 * 1024) {
    const int rc = allow_large_lds(reinterpret_cast<const void*>(kern), LDS);
    if (rc != 0) return rc;
  }
  hipLaunchKernelGGL(kern, dim3(grid_x, 1, (unsigned)batch), dim3(NT), LDS, s, g, epi);
  return launch_status("gemm_kernel");
}

static bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

static int compute_units() {
  static int cus = [] {
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0)
      n = 256;
    return n;
  }();
  return cus;
}

template <typename T, int BM, int BN, int WM, int WN, typename Epi, int NS = 2>
static int launch_fast(GemmArgs g, const Epi& epi, int batch, hipStream_t s) {
  constexpr int NT = WM * WN * kWave;
  constexpr int LDS = fast_lds_bytes<BM, BN, WM, WN, NS>();
  static_assert(LDS <= kLdsPerCu, "tile does not fit in LDS");
  if (describe_only("dma", WM * WN, BM, BN)) return 0;
  g.tiles_m = (g.m + BM - 1) / BM;
  g.tiles_n = (g.n + BN - 1) / BN;
  const int64_t tiles = (int64_t)g.tiles_m * g.tiles_n;
  TTMI_REQUIRE(tiles < (1ll << 30) && batch < 65536, "GEMM grid too large");
  // as many workgroups as stay resident (LDS-limited), a multiple of the XCD count
  const int64_t resident = (int64_t)compute_units() * std::max(1, kLdsPerCu / LDS);
  const unsigned grid_x =
      tiles >= kXcdRemapMinTiles
          ? (unsigned)(std::min(ceil_div(tiles, kNumXcd), std::max<int64_t>(1, resident / kNumXcd)) * kNumXcd)
          : (unsigned)tiles;
  if (!absmax_grid_ok(epi, grid_x, batch)) return launch_fast<T, BM, BN, WM, WN, Epi, NS>(g, without_absmax(epi), batch, s);
  auto kern = gemm_fast_kernel<T, BM, BN, WM, WN, NS, Epi>;
  if (LDS > 64 * 1024) {
    const int rc = allow_large_lds(reinterpret_cast<const void*>(kern), LDS);
    if (rc != 0) return rc;
  }
  hipLaunchKernelGGL(kern, dim3(grid_x, 1, (unsigned)batch), dim3(NT), LDS, s, g, epi);
  return launch_status("gemm_fast_kernel");
}

// Workspace of the split-K path: one buffer per stream, grown on demand, kept for the life of
// the process (work on one stream is ordered, so consecutive GEMMs can share it).
//
// A caller that must not allocate (ttmi_gemm_bias_layer_norm_static) installs a fixed buffer for
// the duration of its call on its thread; then that buffer is handed out, or the request is
// refused when it does not fit, and neither hipMalloc nor hipFree is reached.
struct FixedWorkspace {
  float* ptr = nullptr;
  size_t bytes = 0;
};
static thread_local FixedWorkspace tl_fixed_workspace;

static int splitk_workspace(size_t bytes, hipStream_t s, float** out) {
  *out = nullptr;
  if (tl_fixed_workspace.ptr != nullptr) {
    if (bytes > tl_fixed_workspace.bytes)
      return fail(TTMI_EINVAL, "the K slices of this problem need " + std::to_string(bytes) +
                                   " bytes of partial tiles, more than the static scratch buffer of " +
                                   std::to_string(tl_fixed_workspace.bytes) + " bytes");
    *out = tl_fixed_workspace.ptr;
    return 0;
  }
  struct Slot {
    float* ptr = nullptr;
    size_t bytes = 0;
  };
  static std::mutex mu;
  static std::map<hipStream_t, Slot> slots;
  std::lock_guard<std::mutex> lock(mu);
  Slot& slot = slots[s];
  if (slot.bytes < bytes) {
    if (slot.ptr != nullptr) {
      TTMI_HIP(hipStreamSynchronize(s));
      (void)hipFree(slot.ptr);
      slot = Slot{};
    }
    const size_t want = std::max(bytes, (size_t)8 << 20);
    void* p = nullptr;
    if (hipMalloc(&p, want) != hipSuccess) {
      (void)hipGetLastError();
      return fail(TTMI_ENOMEM, "cannot allocate the split-K workspace");
    }
    slot.ptr = static_cast<float*>(p);
    slot.bytes = want;
  }
  *out = slot.ptr;
  return 0;
}

// Number of K slices for a small problem (1 = do not split): enough workgroups to cover the chip,
// at least four K steps per slice.  A split costs a second launch (4 us for the smallest kernel on
// this chip), which a problem that already has a hundred tiles of 16-bit operands does not win back:
// 128 x 3072 x 768 in fp16 runs 1.3 us faster unsplit, with its epilogue in the GEMM; in fp32 (twice
// the K steps, a quarter of the matrix rate) the same problem is 15 us faster split.
static int pick_splits(int64_t m, int64_t n, int64_t ksteps, int64_t batch, size_t elem_size) {
  const int64_t tiles = ceil_div(m, 64) * ceil_div(n, 64);
  const int64_t most_tiles = elem_size <= 2 ? 64 : 128;
  if (batch != 1 || tiles > most_tiles || ksteps < 8) return 1;
  return (int)std::max<int64_t>(1, std::min<int64_t>({(int64_t)compute_units() / tiles, ksteps / 4, 16}));
}

// The wavefront kernel takes 16-bit problems of at most 128 rows on the [N,K] path (TTMI_WAVE_KERNEL=0 keeps them on
// the 64 x 64 tiles, for A/B timing).
constexpr int kWaveDepth = 4;  // K steps a wavefront keeps in flight: 32 loads of 16 bytes per lane
template <typename T>
static bool wave_kernel_ok(const GemmArgs& g, int batch, bool aligned) {
  if (sizeof(T) != 2 || !aligned || batch != 1 || g.m > 128 || g.k % (kRowBytes / (int)sizeof(T)) != 0) return false;
  return kernel_switch(kSwitchWaveKernel) != 0;
}
// K slices for it: up to two wavefronts per CU, at least four K steps per slice.
static int wave_splits(int64_t m, int64_t n, int64_t ksteps) {
  const int64_t tiles = ceil_div(m, 32) * ceil_div(n, 32);
  return (int)std::max<int64_t>(1, std::min<int64_t>({2 * (int64_t)compute_units() / tiles, ksteps / 4, 16}));
}
static void wave_grid(GemmArgs& g, unsigned* grid_x) {
  g.tiles_m = (g.m + 31) / 32;
  g.tiles_n = (g.n + 31) / 32;
  const int64_t tiles = (int64_t)g.tiles_m * g.tiles_n;
  *grid_x = tiles >= kXcdRemapMinTiles ? (unsigned)(ceil_div(tiles, kNumXcd) * kNumXcd) : (unsigned)tiles;
}
template <typename T, typename Epi>
static int launch_wave(GemmArgs g, const Epi& epi, hipStream_t s) {
  if constexpr (sizeof(T) == 2) {
    if (describe_only("wave", 1, 32, 32)) return 0;
    unsigned grid_x = 0;
    wave_grid(g, &grid_x);
    hipLaunchKernelGGL((gemm_wave_kernel<T, kWaveDepth, Epi>), dim3(grid_x, 1, 1), dim3(kWave), 0, s, g, epi);
  }
  return launch_status("gemm_wave_kernel");
}

// `reduce(ws, slices, vec, stream)` launches the kernel that sums the slices and applies the epilogue.
template <typename T, typename Reduce>
static int launch_splitk(GemmArgs g, int splits, int64_t ksteps, int bk, hipStream_t s, const Reduce& reduce) {
  constexpr int kTile = 64, kWaveTile = 32;  // tile edge of the LDS-tiled and of the one-wavefront form
  const bool wave = wave_kernel_ok<T>(g, 1, true);  // callers come here with aligned operands and one problem
  if (wave) splits = std::max(2, wave_splits(g.m, g.n, ksteps));
  g.k_chunk = (int)ceil_div(ksteps, splits) * bk;
  const int used = (int)ceil_div(g.k, g.k_chunk);  // slices that actually hold part of K: what is launched
  if (describe_only(wave ? "wave" : "reg", wave ? 1 : 4, wave ? kWaveTile : kTile, wave ? kWaveTile : kTile, used)) return 0;
  const size_t bytes = (size_t)used * g.m * g.n * sizeof(float);
  float* ws = nullptr;
  {
    const int rc = splitk_workspace(bytes, s, &ws);
    if (rc != 0) return rc;
  }
  const bool vec = g.n % 4 == 0;
  EpiPartial part{ws, (int64_t)g.m * g.n, g.n, vec};
  if constexpr (sizeof(T) == 2) {
    if (wave) {
      unsigned wgrid = 0;
      wave_grid(g, &wgrid);
      hipLaunchKernelGGL((gemm_wave_kernel<T, kWaveDepth, EpiPartial>), dim3(wgrid, (unsigned)used, 1), dim3(kWave), 0, s, g, part);
      reduce(ws, used, vec, s);
      return launch_status("gemm_wave_splitk");
    }
  }
  g.tiles_m = (g.m + kTile - 1) / kTile;
  g.tiles_n = (g.n + kTile - 1) / kTile;
  const int64_t tiles = (int64_t)g.tiles_m * g.tiles_n;
  constexpr int LDS = 2 * (kTile + kTile) * kRowBytes;
  const unsigned grid_x = tiles >= kXcdRemapMinTiles ? (unsigned)(ceil_div(tiles, kNumXcd) * kNumXcd) : (unsigned)tiles;
  hipLaunchKernelGGL((gemm_kernel<T, kTile, kTile, 2, 2, false, true, 2, EpiPartial>), dim3(grid_x, (unsigned)used, 1), dim3(256), LDS, s,
                     g, part);
  reduce(ws, used, vec, s);
  return launch_status("gemm_splitk");
}

// Split-K on the DMA kernel with 128x128 tiles, for mid-size problems whose tiles do not fill the chip
// (M = 2560, N = 768, K = 3072: 120 tiles, 48 K steps each).
template <typename T, typename Reduce>
static int launch_fast_splitk(GemmArgs g, int splits, int64_t ksteps, int bk, hipStream_t s, const Reduce& reduce) {
  constexpr int kTile = 128;
  g.k_chunk = (int)ceil_div(ksteps, splits) * bk;
  const int used = (int)ceil_div(g.k, g.k_chunk);  // slices that actually hold part of K: what is launched
  if (describe_only("dma", 4, kTile, kTile, used)) return 0;
  const size_t bytes = (size_t)used * g.m * g.n * sizeof(float);
  float* ws = nullptr;
  {
    const int rc = splitk_workspace(bytes, s, &ws);
    if (rc != 0) return rc;
  }
  g.tiles_m = (g.m + kTile - 1) / kTile;
  g.tiles_n = (g.n + kTile - 1) / kTile;
  const int64_t tiles = (int64_t)g.tiles_m * g.tiles_n;
  const bool vec = g.n % 4 == 0;
  EpiPartial part{ws, (int64_t)g.m * g.n, g.n, vec};
  constexpr int LDS = fast_lds_bytes<kTile, kTile, 2, 2>();
  auto kern = gemm_fast_kernel<T, kTile, kTile, 2, 2, 2, EpiPartial>;
  {
    const int rc = allow_large_lds(reinterpret_cast<const void*>(kern), LDS);
    if (rc != 0) return rc;
  }
  // one workgroup per (tile, slice): the persistent loop runs once
  const unsigned grid_x = tiles >= kXcdRemapMinTiles ? (unsigned)(ceil_div(tiles, kNumXcd) * kNumXcd) : (unsigned)tiles;
  hipLaunchKernelGGL(kern, dim3(grid_x, (unsigned)used, 1), dim3(256), LDS, s, g, part);
  reduce(ws, used, vec, s);
  return launch_status("gemm_fast_splitk");
}

// The ordinary reduction: sum the slices, then the epilogue the unsplit kernel would have applied.
template <typename Epi>
struct ReduceWithEpilogue {
  Epi epi;
  int m, n;
  void operator()(const float* ws, int slices, bool vec, hipStream_t s) const {
    const int64_t items = (int64_t)m * ((n + 7) / 8);
    hipLaunchKernelGGL((splitk_reduce_kernel<Epi>), dim3((unsigned)ceil_div(items, 256)), dim3(256), 0, s, ws, slices, m, n, vec, epi);
  }
};

// Tile configurations of the fast path and a cost model to pick one.  With t = tile area /
// efficiency as the time of one tile on an otherwise idle CU, and `per_cu` workgroups of that
// size resident per CU (they then share its MFMA pipes):
//   time ~ full_rounds * per_cu * t  +  ceil(remaining_tiles / CUs) * t
// Large tiles reuse LDS operands best (efficiency 1.0 for 256x256) but quantise badly when the
// tile count is a small non-multiple of the 256 CUs, e.g. N = 768 at M = 32768: 384 tiles of
// 256x256 are 1.5 rounds, 512 tiles of 256x192 are exactly 2.  Problems with few tiles take
// the smallest tile: they are latency-bound and want as many CUs as possible.
struct TileConfig {
  int bm, bn, per_cu;
  float eff;
};
constexpr TileConfig kTileConfigs[] = {
    {256, 256, 1, 1.00f}, {256, 192, 1, 0.93f}, {256, 128, 1, 0.82f}, {128, 128, 2, 0.62f}, {64, 64, 4, 0.30f}};

static double tile_cost(const TileConfig& c, int64_t m, int64_t n, int64_t batch) {
  const int64_t tiles = ceil_div(m, c.bm) * ceil_div(n, c.bn) * batch;
  const int64_t slots = (int64_t)compute_units() * c.per_cu;
  const int64_t full = tiles / slots, rem = tiles % slots;
  const double t = (double)c.bm * c.bn / c.eff;
  return (double)full * c.per_cu * t + (double)ceil_div(rem, compute_units()) * t;
}

// fp32: the matrix pipe is sixteen times slower than for 16-bit operands and bounds every tile size, so what counts is
// how evenly the tiles load the CUs (all wavefronts resident on a CU share its four SIMDs), and the small tiles lose
// little: efficiencies fitted to a sweep of M = 800 ... 16384 by N, K = 768 / 3072 (4000 x 768 x 3072: 175 us on
// 64 x 64 tiles, three per CU, against 233 us on 128 x 128, one on three CUs of four).
constexpr float kTileEff32[] = {0.88f, 0.85f, 0.82f, 0.78f, 0.74f};
static double tile_cost32(int i, int64_t m, int64_t n, int64_t batch) {
  const TileConfig& c = kTileConfigs[i];
  const int64_t tiles = ceil_div(m, c.bm) * ceil_div(n, c.bn) * batch;
  return (double)ceil_div(tiles, compute_units()) * c.bm * c.bn / kTileEff32[i];
}

static int pick_tile(int64_t m, int64_t n, int64_t batch, double* cost_out = nullptr, size_t elem_size = 2) {
  int best = 0;
  double best_cost = 1e300;
  for (int i = 0; i < (int)(sizeof(kTileConfigs) / sizeof(kTileConfigs[0])); ++i) {
    const double cost = elem_size == 4 ? tile_cost32(i, m, n, batch) : tile_cost(kTileConfigs[i], m, n, batch);
    if (cost < best_cost) {
      best_cost = cost;
      best = i;
    }
  }
  if (cost_out != nullptr) *cost_out = best_cost;
  return best;
}

// Hook for the one-wavefront-per-SIMD kernel of gemm_w4.h, which specialises it for the element types and
// epilogues it serves: wanted() says whether that kernel should take the problem, launch() runs it.
template <typename T, typename Epi, typename Enable = void>
struct LargeTileKernel {
  static bool wanted(const GemmArgs&, const Epi&, int, bool) { return false; }
  static int launch(const GemmArgs&, const Epi&, hipStream_t) { return 0; }
};

// Whether (and how) a problem on the [N,K]-weights path is cut along K.
enum class SplitKind { kNone, kSmallTiles, kDmaTiles };
struct SplitPlan {
  SplitKind kind;
  int splits;
};
template <typename T>
static SplitPlan plan_split(int64_t m, int64_t n, int64_t k, int64_t batch, bool aligned) {
  constexpr int BK = kRowBytes / sizeof(T);
  if (!aligned || k % BK != 0 || batch != 1) return {SplitKind::kNone, 1};
  const int64_t ksteps = k / BK;
  const int tile = pick_tile(m, n, batch, nullptr, sizeof(T));
  if (tile == 4) {
    const int splits = pick_splits(m, n, ksteps, batch, sizeof(T));
    if (splits > 1) return {SplitKind::kSmallTiles, splits};
    if (sizeof(T) == 4) {
      // fp32 with more tiles than that: whole rounds of tiles over the CUs are what the launch costs, and a last round
      // that is nearly empty (1600 x 768: 300 tiles, two rounds for 1.17 CUs' worth) is repaired by cutting K so that
      // the slices fill the rounds.  Estimate in microseconds: matrix time of the rounds at the fitted efficiency plus
      // the pass that sums the slices (their bytes at 4 TB/s and a launch); partial tiles of at most 32 MiB.
      const int64_t tiles = ceil_div(m, 64) * ceil_div(n, 64);
      const double per_round = 64.0 * 64.0 * 2.0 * (double)k / (157.3e6 / compute_units() * kTileEff32[4]);  // us, whole K
      const double uncut = (double)ceil_div(tiles, compute_units()) * per_round;
      double best = uncut;
      int best_splits = 1;
      for (int sp = 2; sp <= 8 && ksteps / sp >= 4 && (int64_t)sp * m * n * 4 <= (32ll << 20); ++sp) {
        const double reduce = (double)(sp + 1) * m * n * 4 / 4e6 + 4.0;
        const double t = (double)ceil_div(tiles * sp, compute_units()) * per_round / sp + reduce;
        if (t < best) {
          best = t;
          best_splits = sp;
        }
      }
      if (best < 0.9 * uncut) return {SplitKind::kSmallTiles, best_splits};
    }
  }
  // (the cost model knows nothing of K: a few hundred rows by 768 columns by K = 3072 are 150 tiles of 64 x 64, too many
  // for the small split, each a serial chain of 48 K steps; cut on 128 x 128 tiles they are 250 workgroups of 8 steps)
  // (not fp32: there the 64 x 64 tiles the model picks for such a shape already load every SIMD)
  if (sizeof(T) != 4 && (tile == 3 || tile == 4)) {
    const int64_t t128 = ceil_div(m, 128) * ceil_div(n, 128);
    if (t128 <= compute_units() / 2 && ksteps >= 16) {
      // one and a half workgroups per CU: with two (four slices at 2560 x 768, five at 2048 x 768) the extra fp32
      // partial tiles cost more than the shorter K loops save (20 x 128 tokens -1.3 %, ALBERT 8 x 256 -3.3 % with one slice less)
      const int splits = (int)std::min<int64_t>({3 * (int64_t)compute_units() / (2 * t128), ksteps / 8, 8});
      if (splits > 1) return {SplitKind::kDmaTiles, splits};
    }
  }
  return {SplitKind::kNone, 1};
}

template <typename T, bool B_KN, typename Epi>
static int launch_gemm(GemmArgs g, const Epi& epi, int batch, bool aligned, hipStream_t s) {
  if (g.m <= 0 || g.n <= 0 || batch <= 0) return 0;
  TTMI_REQUIRE(g.k > 0, "K must be positive");
  auto tiles = [&](int bm, int bn) { return (int64_t)ceil_div(g.m, bm) * ceil_div(g.n, bn) * batch; };
  if (!B_KN) {
    constexpr int BK = kRowBytes / sizeof(T);
    if (aligned && g.k % BK == 0) {
      bool column_pass = false;
      if constexpr (HasColumnPass<Epi>::value) column_pass = epi.v_pitch > 0;
      if (LargeTileKernel<T, Epi>::wanted(g, epi, batch, aligned)) return LargeTileKernel<T, Epi>::launch(g, epi, s);
      switch (pick_tile(g.m, g.n, batch, nullptr, sizeof(T))) {
        case 0: return launch_fast<T, 256, 256, 2, 4, Epi>(g, epi, batch, s);
        case 1: return launch_fast<T, 256, 192, 4, 2, Epi>(g, epi, batch, s);
        case 2: return launch_fast<T, 256, 128, 4, 2, Epi>(g, epi, batch, s);
        case 3: {
          if constexpr (std::is_same<typename Epi::Acc, float>::value) {
            const SplitPlan plan = column_pass ? SplitPlan{SplitKind::kNone, 1} : plan_split<T>(g.m, g.n, g.k, batch, aligned);
            if (plan.kind == SplitKind::kDmaTiles)
              return launch_fast_splitk<T>(g, plan.splits, g.k / BK, BK, s, ReduceWithEpilogue<Epi>{epi, g.m, g.n});
          }
          // 128 x 128 tiles on at most half the CUs and a K too short to cut: 128 x 64 tiles put twice as many CUs
          // to work (2560 x 768 x 768: 240 tiles in one round, 9 us against 11)
          if (batch == 1 && tiles(128, 128) <= compute_units() / 2 && tiles(128, 64) <= compute_units())
            return launch_fast<T, 128, 64, 2, 2, Epi, 4>(g, epi, batch, s);
          return launch_fast<T, 128, 128, 2, 2, Epi>(g, epi, batch, s);
        }
        // small problems are latency-bound: the register-staged kernel hides the global latency
        // of a one-step prefetch better than the DMA path does with a tiny tile
        default: {
          if constexpr (std::is_same<typename Epi::Acc, float>::value) {
            const SplitPlan plan = column_pass ? SplitPlan{SplitKind::kNone, 1} : plan_split<T>(g.m, g.n, g.k, batch, aligned);
            if (plan.kind == SplitKind::kSmallTiles)
              return launch_splitk<T>(g, plan.splits, g.k / BK, BK, s, ReduceWithEpilogue<Epi>{epi, g.m, g.n});
            if (plan.kind == SplitKind::kDmaTiles)
              return launch_fast_splitk<T>(g, plan.splits, g.k / BK, BK, s, ReduceWithEpilogue<Epi>{epi, g.m, g.n});
            if (wave_kernel_ok<T>(g, batch, aligned)) return launch_wave<T>(g, epi, s);
          }
          return launch_config<T, 64, 64, 2, 2, false, true, Epi>(g, epi, batch, s);
        }
      }
    }
    if (aligned) {
      if (tiles(128, 128) >= 200) return launch_config<T, 128, 128, 2, 2, false, true, Epi>(g, epi, batch, s);
      return launch_config<T, 64, 64, 2, 2, false, true, Epi>(g, epi, batch, s);
    }
    return launch_config<T, 64, 64, 2, 2, false, false, Epi>(g, epi, batch, s);
  } else {
    if (aligned) {
      if (tiles(128, 128) >= 200 && g.n >= 96) return launch_config<T, 128, 128, 2, 2, true, true, Epi>(g, epi, batch, s);
      return launch_config<T, 64, 64, 2, 2, true, true, Epi>(g, epi, batch, s);
    }
    return launch_config<T, 64, 64, 2, 2, true, false, Epi>(g, epi, batch, s);
  }
}

template <typename T>
static int gemm_alpha_beta(const void* a, const void* b, void* c, int64_t m, int64_t n, int64_t k, int64_t lda,
                           int64_t ldb, int64_t ldc, int inner, int64_t a_outer, int64_t a_inner,
                           int64_t b_outer, int64_t b_inner, int64_t c_outer, int64_t c_inner, int64_t batch,
                           int trans_b, float alpha, float beta, hipStream_t s) {
  TTMI_REQUIRE(m < (1ll << 31) && n < (1ll << 31) && k < (1ll << 31), "dimension too large");
  GemmArgs g{};
  g.a = (const char*)a;
  g.b = (const char*)b;
  g.m = (int)m; g.n = (int)n; g.k = (int)k;
  g.lda = lda; g.ldb = ldb;
  g.inner = inner;
  g.a_outer = a_outer; g.a_inner = a_inner; g.b_outer = b_outer; g.b_inner = b_inner;
  constexpr int KPC = 16 / sizeof(T);
  const bool c_vec = aligned16(c) && ldc % KPC == 0 && c_outer % KPC == 0 && c_inner % KPC == 0;
  EpiAlphaBeta<T> epi{(T*)c, ldc, c_outer, c_inner, inner, alpha, beta, c_vec};
  auto mult = [](int64_t v) { return v % KPC == 0; };
  bool aligned = aligned16(a) && aligned16(b) && mult(lda) && mult(ldb) && mult(a_outer) && mult(a_inner) &&
                 mult(b_outer) && mult(b_inner);
  if (trans_b) {
    aligned = aligned && mult(k);
    return launch_gemm<T, false>(g, epi, (int)batch, aligned, s);
  }
  aligned = aligned && mult(k) && mult(n);
  return launch_gemm<T, true>(g, epi, (int)batch, aligned, s);
}

}  // namespace ttmi
