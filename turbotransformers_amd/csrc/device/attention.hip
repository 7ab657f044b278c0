// Fused self-attention for head_dim 64, fp16/bf16:  out = softmax(scale * Q K^T + mask) V
// in one kernel, without materialising the [B,h,S,S] score tensor in HBM.  It replaces the
// batch_gemm3 -> ApplyMaskAndSoftmax -> batch_gemm4 -> TransposeForScore chain of
// layers/multi_headed_attention.cpp:323-354 whenever the caller does not ask for the
// attention probabilities (then only Q, K, V are read and the merged context is written:
// 4*T*H elements instead of ~2*B*h*S^2).
//
// Work split: one workgroup = 4 wavefronts = 128 query rows of one (batch, head); a wavefront
// owns 32 queries.  K/V advance in tiles of 64 keys staged in LDS (K row-major and
// XOR-swizzled like the GEMM operands, V transposed to [d][key]).
//
// MFMA formulation (v_mfma_f32_32x32x16): scores are computed TRANSPOSED,
//     St[key, query] = K_tile[key, :] . Q[query, :]      (A = K from LDS, B = Q from registers)
// so a lane holds ONE query column (lane%32) and 16 key rows.  Row statistics of the online
// softmax are then lane-local plus one exchange between the two half-waves, and the
// probabilities, still in accumulator registers, are already laid out as the B operand of
//     Ot[d, query] += Vt[d, keys] . Pt[keys, query]      (A = V^T from LDS, B = P from registers)
// because accumulator registers 8kk..8kk+7 of a lane are exactly the 8 keys that half-wave
// feeds to MFMA kk.  No cross-lane shuffles of P, no LDS round trip for P.
// exp() is evaluated as exp2 with log2(e) folded into the scale and the mask.
#include "common.h"

namespace ttmi {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef _Float16 halfx8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

struct __attribute__((may_alias)) alignas(16) Chunk16 {
  uint32_t w[4];
};
struct __attribute__((may_alias)) alignas(8) Chunk8 {
  uint32_t w[2];
};

template <typename T>
__device__ __forceinline__ floatx16 mma16(const Chunk16& a, const Chunk16& b, floatx16 c);
template <>
__device__ __forceinline__ floatx16 mma16<f16>(const Chunk16& a, const Chunk16& b, floatx16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(halfx8, a), __builtin_bit_cast(halfx8, b), c, 0, 0, 0);
}
template <>
__device__ __forceinline__ floatx16 mma16<bf16>(const Chunk16& a, const Chunk16& b, floatx16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
}

template <typename T>
__device__ __forceinline__ uint32_t pack2(float lo, float hi) {
  const T a = from_float<T>(lo), b = from_float<T>(hi);
  uint16_t ua, ub;
  __builtin_memcpy(&ua, &a, 2);
  __builtin_memcpy(&ub, &b, 2);
  return (uint32_t)ua | ((uint32_t)ub << 16);
}

constexpr int kD = 64;          // head dim
constexpr int kBQ = 128;        // queries per workgroup
constexpr int kBKV = 64;        // keys per LDS tile
constexpr int kVtPitch = kBKV + 4;  // halfs per V^T row (8-byte aligned rows, spreads banks)
constexpr float kNegBig = -1.0e30f;

template <typename T, bool PACKED>
__global__ __launch_bounds__(256) void fused_attention_kernel(const T* __restrict__ q, const T* __restrict__ k,
                                                              const T* __restrict__ v, const float* __restrict__ mask,
                                                              T* __restrict__ out, const int32_t* __restrict__ cu,
                                                              int heads, int seq, float scale_log2e) {
  // one LDS block: [2 x K tile | 2 x V^T tile | 2 x mask]; the front is reused for the output tile
  constexpr int kKBytes = kBKV * 128, kVtBytes = kD * kVtPitch * (int)sizeof(T);
  __shared__ __align__(16) char smem[2 * kKBytes + 2 * kVtBytes + 2 * kBKV * 4];
  static_assert(4 * 32 * (kD + 8) * sizeof(T) <= 2 * kKBytes + 2 * kVtBytes, "output staging must fit in the tile buffers");
  auto k_lds = [&](int stage) { return smem + stage * kKBytes; };
  auto vt_lds = [&](int stage) { return reinterpret_cast<T*>(smem + 2 * kKBytes + stage * kVtBytes); };
  auto mask_lds = [&](int stage) { return reinterpret_cast<float*>(smem + 2 * kKBytes + 2 * kVtBytes) + stage * kBKV; };

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int lrow = lane & 31, lhalf = lane >> 5;
  const int bh = blockIdx.y, b = bh / heads, head = bh - b * heads;
  const int q0 = blockIdx.x * kBQ + wave * 32;

  int kv_len = seq, out_row0 = b * seq;
  if (PACKED) {
    kv_len = cu[b + 1] - cu[b];
    out_row0 = cu[b];
    if ((int)blockIdx.x * kBQ >= kv_len) return;  // whole workgroup is padding
  }
  const int q_len = kv_len;  // self attention: as many queries as keys

  const T* qb = q + (int64_t)bh * seq * kD;
  const T* kb = k + (int64_t)bh * seq * kD;
  const T* vb = v + (int64_t)bh * seq * kD;

  // Q fragments: B operand, lane = (query lrow, k-chunk by lhalf); 4 MFMA k-steps cover d = 64.
  Chunk16 qf[4];
  {
    const int qi = q0 + lrow;
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) {
      if (qi < seq) qf[kk] = *reinterpret_cast<const Chunk16*>(qb + (int64_t)qi * kD + (2 * kk + lhalf) * 8);
      else qf[kk] = Chunk16{{0u, 0u, 0u, 0u}};
    }
  }

  floatx16 ot[2];
#pragma unroll
  for (int t = 0; t < 2; ++t)
#pragma unroll
    for (int e = 0; e < 16; ++e) ot[t][e] = 0.f;
  float m_run = kNegBig, l_run = 0.f;

  auto load_tile = [&](int tile, int stage) {
    const int key0 = tile * kBKV;
    // K: 64 keys x 8 chunks; thread c -> (key c>>3, chunk c&7): 128-byte rows, coalesced
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int c = tid + i * 256;
      const int key = c >> 3, ch = c & 7;
      Chunk16 x{{0u, 0u, 0u, 0u}};
      if (key0 + key < kv_len) x = *reinterpret_cast<const Chunk16*>(kb + (int64_t)(key0 + key) * kD + ch * 8);
      *reinterpret_cast<Chunk16*>(k_lds(stage) + key * 128 + ((ch ^ ((key >> 1) & 7)) << 4)) = x;
    }
    // V: thread -> (key tid&63, d-chunk (tid>>6) + 4i); scattered into V^T[d][key] so that lanes
    // write consecutive halfs of one row (no bank conflicts)
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int key = tid & 63, dch = (tid >> 6) + 4 * i;
      Vec<T, 8> x;
      if (key0 + key < kv_len) {
        x = load_vec<T, 8>(vb + (int64_t)(key0 + key) * kD + dch * 8);
      } else {
#pragma unroll
        for (int j = 0; j < 8; ++j) x.v[j] = from_float<T>(0.f);
      }
#pragma unroll
      for (int j = 0; j < 8; ++j) vt_lds(stage)[(dch * 8 + j) * kVtPitch + key] = x.v[j];
    }
    if (tid < kBKV) {
      const int key = key0 + tid;
      float mv = kNegBig;
      if (key < kv_len) mv = mask ? mask[(int64_t)b * seq + key] * 1.4426950408889634f : 0.f;
      mask_lds(stage)[tid] = mv;
    }
  };

  const int tiles = (kv_len + kBKV - 1) / kBKV;
  const bool wave_active = q0 < q_len;
  load_tile(0, 0);
  __syncthreads();
  for (int tile = 0; tile < tiles; ++tile) {
    const int stage = tile & 1;
    if (tile + 1 < tiles) load_tile(tile + 1, stage ^ 1);
    if (wave_active) {
#pragma unroll
      for (int sub = 0; sub < 2; ++sub) {  // two 32-key sub-tiles
        const int sk = sub * 32;
        floatx16 st;
#pragma unroll
        for (int e = 0; e < 16; ++e) st[e] = 0.f;
#pragma unroll
        for (int kk = 0; kk < 4; ++kk) {
          const int key = sk + lrow;
          const Chunk16 kf = *reinterpret_cast<const Chunk16*>(k_lds(stage) + key * 128 + (((2 * kk + lhalf) ^ ((key >> 1) & 7)) << 4));
          st = mma16<T>(kf, qf[kk], st);
        }
        // st[e] = score of (key sk + 8*(e/4) + 4*lhalf + e%4, query lrow)
        float mx = kNegBig;
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          const int key = sk + 8 * (e / 4) + 4 * lhalf + (e % 4);
          st[e] = st[e] * scale_log2e + mask_lds(stage)[key];
          mx = fmaxf(mx, st[e]);
        }
        mx = fmaxf(mx, __shfl_xor(mx, 32, kWave));
        const float m_new = fmaxf(m_run, mx);
        const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
        m_run = m_new;
        float psum = 0.f;
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          st[e] = __builtin_amdgcn_exp2f(st[e] - m_new);
          psum += st[e];
        }
        l_run = l_run * alpha + psum;
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
          for (int e = 0; e < 16; ++e) ot[t][e] *= alpha;
#pragma unroll
        for (int kk = 0; kk < 2; ++kk) {
          Chunk16 pf;
#pragma unroll
          for (int w = 0; w < 4; ++w) pf.w[w] = pack2<T>(st[8 * kk + 2 * w], st[8 * kk + 2 * w + 1]);
#pragma unroll
          for (int t = 0; t < 2; ++t) {
            const T* row = vt_lds(stage) + (t * 32 + lrow) * kVtPitch + sk + 16 * kk + 4 * lhalf;
            const Chunk8 lo = *reinterpret_cast<const Chunk8*>(row);
            const Chunk8 hi = *reinterpret_cast<const Chunk8*>(row + 8);
            const Chunk16 vf{{lo.w[0], lo.w[1], hi.w[0], hi.w[1]}};
            ot[t] = mma16<T>(vf, pf, ot[t]);
          }
        }
      }
    }
    __syncthreads();
  }

  // normalise and write: ot[t][e] = O[query lrow][d = 32t + 8*(e/4) + 4*lhalf + e%4]
  const float l_tot = l_run + __shfl_xor(l_run, 32, kWave);
  const float inv = 1.0f / l_tot;
  // stage the wavefront's 32x64 tile in LDS (K buffers are free now) to store 128-byte rows
  T* stage_o = reinterpret_cast<T*>(smem) + wave * (32 * (kD + 8));
#pragma unroll
  for (int t = 0; t < 2; ++t)
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      Chunk8 c;
      c.w[0] = pack2<T>(ot[t][4 * g] * inv, ot[t][4 * g + 1] * inv);
      c.w[1] = pack2<T>(ot[t][4 * g + 2] * inv, ot[t][4 * g + 3] * inv);
      *reinterpret_cast<Chunk8*>(stage_o + lrow * (kD + 8) + t * 32 + 8 * g + 4 * lhalf) = c;
    }
  const int hd = heads * kD;
#pragma unroll
  for (int p = 0; p < 4; ++p) {
    const int r = p * 8 + (lane >> 3), cchunk = lane & 7;
    const int qi = q0 + r;
    if (qi < q_len && qi < seq) {
      const Chunk16 x = *reinterpret_cast<const Chunk16*>(stage_o + r * (kD + 8) + cchunk * 8);
      *reinterpret_cast<Chunk16*>(out + ((int64_t)(out_row0 + qi)) * hd + head * kD + cchunk * 8) = x;
    }
  }
}

}  // namespace ttmi

using namespace ttmi;

extern "C" {

int ttmi_fused_attention(const void* q, const void* k, const void* v, const float* mask, void* out,
                         const int32_t* cu_seqlens, int64_t batch, int64_t heads, int64_t seq, int64_t head_dim,
                         float scale, int dtype, void* stream) {
  TTMI_REQUIRE(q && k && v && out, "null tensor");
  TTMI_REQUIRE(head_dim == kD, "fused attention is built for head_dim 64");
  TTMI_REQUIRE(dtype == TTMI_F16 || dtype == TTMI_BF16, "fused attention is built for fp16 / bf16");
  TTMI_REQUIRE(batch > 0 && heads > 0 && seq > 0 && batch * heads < 65536 && seq < (1 << 24), "bad shape");
  uintptr_t bits = reinterpret_cast<uintptr_t>(q) | reinterpret_cast<uintptr_t>(k) | reinterpret_cast<uintptr_t>(v) |
                   reinterpret_cast<uintptr_t>(out);
  TTMI_REQUIRE((bits & 15) == 0, "tensors must be 16-byte aligned");
  const dim3 grid((unsigned)ceil_div(seq, kBQ), (unsigned)(batch * heads));
  const float sl2 = scale * 1.4426950408889634f;
  hipStream_t s = (hipStream_t)stream;
#define TTMI_FA_LAUNCH(T, PACKED)                                                                              \
  hipLaunchKernelGGL((fused_attention_kernel<T, PACKED>), grid, dim3(256), 0, s, (const T*)q, (const T*)k,     \
                     (const T*)v, mask, (T*)out, cu_seqlens, (int)heads, (int)seq, sl2)
  if (dtype == TTMI_F16) {
    if (cu_seqlens) TTMI_FA_LAUNCH(f16, true); else TTMI_FA_LAUNCH(f16, false);
  } else {
    if (cu_seqlens) TTMI_FA_LAUNCH(bf16, true); else TTMI_FA_LAUNCH(bf16, false);
  }
#undef TTMI_FA_LAUNCH
  return launch_status("fused_attention");
}

}  // extern "C"
