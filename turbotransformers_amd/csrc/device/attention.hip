// Fused self-attention for head_dim 64, fp16/bf16:  out = softmax(scale * Q K^T + mask) V
// in one kernel, without materialising the [B,h,S,S] score tensor in HBM.  It replaces the
// batch_gemm3 -> ApplyMaskAndSoftmax -> batch_gemm4 -> TransposeForScore chain of
// layers/multi_headed_attention.cpp:323-354 whenever the caller does not ask for the
// attention probabilities (then only Q, K, V are read and the merged context is written:
// 4*T*H elements instead of ~2*B*h*S^2).
//
// Work split: one workgroup = NW wavefronts = 32 NW query rows of one (batch, head); a wavefront
// owns 32 queries.  Every workgroup streams all keys and values of its head through LDS, and what a CU can
// fetch (about 45 GB/s) is what bounds the kernel -- with the loads and LDS stores of the tiles removed it runs
// 29 % faster, with the exponentials or either matrix product removed 5 % -- so long sequences take eight
// wavefronts (256 queries) per workgroup, which halves the bytes fetched per query; up to 128 tokens take four.  K/V advance in tiles of 64 keys staged in LDS: K row-major [key][d], V
// transposed [d][key], both in 128-byte rows XOR-swizzled like the GEMM operands.  V may be
// given already transposed ([B,h,d,pitch], written that way by the QKV GEMM epilogue); then a
// V tile is copied in 8-byte pieces, otherwise it is scattered element by element.
//
// MFMA formulation (v_mfma_f32_32x32x16): scores are computed TRANSPOSED,
//     St[key, query] = K_tile[key, :] . Q[query, :]      (A = K from LDS, B = Q from registers)
// so a lane holds ONE query column (lane%32) and 16 key rows.  Row statistics of the online
// softmax are then lane-local plus one exchange between the two half-waves, and the
// probabilities, still in accumulator registers, are already laid out as the B operand of
//     Ot[d, query] += Vt[d, keys] . Pt[keys, query]      (A = V^T from LDS, B = P from registers)
// because accumulator registers 8kk..8kk+7 of a lane are exactly the 8 keys that half-wave
// feeds to MFMA kk.  No cross-lane shuffles of P, no LDS round trip for P.
// exp() is evaluated as exp2; the mask (divided by the scale) seeds the score accumulators and
// scale*log2(e) is applied inside the exp2 argument, so no separate scale/mask pass exists.
#include <cstdlib>

#include "common.h"

namespace ttmi {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef _Float16 halfx8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

typedef uint32_t u32x4 __attribute__((ext_vector_type(4), may_alias));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2), may_alias));

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

typedef float floatx2 __attribute__((ext_vector_type(2)));
typedef _Float16 halfx2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));

// Two floats -> one packed register (round to nearest even): v_cvt_pk_{f16,bf16}_f32.
template <typename T>
__device__ __forceinline__ uint32_t pack2(float lo, float hi);
template <>
__device__ __forceinline__ uint32_t pack2<f16>(float lo, float hi) {
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(floatx2{lo, hi}, halfx2));
}
template <>
__device__ __forceinline__ uint32_t pack2<bf16>(float lo, float hi) {
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(floatx2{lo, hi}, bf16x2));
}

// acc + lo + hi of a packed pair (v_dot2c_f32_*): the softmax denominator is summed from the
// ROUNDED probabilities, the same values the P.V MFMA consumes.
template <typename T>
__device__ __forceinline__ float add_pair(uint32_t p, float acc);
template <>
__device__ __forceinline__ float add_pair<f16>(uint32_t p, float acc) {
  return __builtin_amdgcn_fdot2(__builtin_bit_cast(halfx2, p), halfx2{(_Float16)1.0f, (_Float16)1.0f}, acc, false);
}
template <>
__device__ __forceinline__ float add_pair<bf16>(uint32_t p, float acc) {
  return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, p), bf16x2{(__bf16)1.0f, (__bf16)1.0f}, acc, false);
}

constexpr int kD = 64;          // head dim
constexpr int kBKV = 64;        // keys per LDS tile
constexpr float kNegBig = -1.0e30f;
// log2 of the largest probability tolerated before the running maximum is moved.  bf16 keeps the
// exact maximum: with 8 mantissa bits a dominant probability of exactly 1.0 is worth keeping exact.
template <typename T>
constexpr float kSlack = sizeof(T) == 2 && !std::is_same<T, bf16>::value ? 8.0f : 0.0f;

// Position of a key inside its group of 16 in an LDS V^T row.  A lane of the P.V MFMA holds the
// probabilities of keys {4h..4h+3, 8+4h..8+4h+3} (h = lane/32) of the group; storing the group as
// [0-3, 8-11, 4-7, 12-15] makes those 8 keys one 16-byte read.
__device__ __forceinline__ int vt_pos(int within16) {
  return (within16 & 3) | ((within16 & 4) << 1) | ((within16 & 8) >> 1);
}

// One 64-key tile: kt = K tile ([key][d], 128-byte rows, swizzled), vt = V^T tile ([d][key], likewise), mk = additive
// mask of its 64 keys divided by the score scale.  m_run is kept in raw score units; the softmax scale and log2(e)
// are applied inside the exp2 argument: p = exp2(s*c - m*c), c = scale*log2(e).  k_off: the lane's four fragment
// offsets inside a 32-row block (see the kernels).
template <typename T>
__device__ __forceinline__ void attention_tile(const char* kt, const char* vt, const float* mk, const Chunk16 (&qf)[4],
                                               const int (&k_off)[4], int lhalf, float scale_log2e, floatx16 (&ot)[2],
                                               float& m_run, float& l_run) {
#pragma unroll
  for (int sub = 0; sub < 2; ++sub) {  // two 32-key sub-tiles
    const int sk = sub * 32;
    // st[e] = score of (key sk + 8*(e/4) + 4*lhalf + e%4, query lrow), seeded with mask/scale
    floatx16 st;
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const float4 mv = *reinterpret_cast<const float4*>(mk + sk + 8 * g + 4 * lhalf);
      st[4 * g] = mv.x, st[4 * g + 1] = mv.y, st[4 * g + 2] = mv.z, st[4 * g + 3] = mv.w;
    }
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) {
      const Chunk16 kf = *reinterpret_cast<const Chunk16*>(kt + sk * 128 + k_off[kk]);
      st = mma16<T>(kf, qf[kk], st);
    }
    float mx = st[0];
#pragma unroll
    for (int e = 1; e < 16; ++e) mx = fmaxf(mx, st[e]);
    {
      // the other half-wavefront holds the remaining 16 keys of this query: exchange through
      // v_permlane32_swap (two VALU instructions) instead of an LDS permute and its wait
      const auto sw = __builtin_amdgcn_permlane32_swap(__builtin_bit_cast(unsigned, mx), __builtin_bit_cast(unsigned, mx), false, false);
      mx = fmaxf(__builtin_bit_cast(float, sw[0]), __builtin_bit_cast(float, sw[1]));
    }
    // Lazy running maximum: the reference point m_run only moves when some query of the
    // wavefront would otherwise see exp2 arguments above kSlack (fp16: probabilities up to 2^kSlack are
    // as precise as smaller ones and the final division by the row sum cancels the choice of
    // m_run), so the rescaling of the 32 output accumulators is skipped for most tiles.
    if (__any((mx - m_run) * scale_log2e > kSlack<T>)) {
      const float m_new = fmaxf(m_run, mx);
      const float alpha = __builtin_amdgcn_exp2f((m_run - m_new) * scale_log2e);
      m_run = m_new;
      l_run *= alpha;
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int e = 0; e < 16; ++e) ot[t][e] *= alpha;
    }
    const float neg_m = -m_run * scale_log2e;
    Chunk16 pf[2];
    float psum = 0.f;
#pragma unroll
    for (int w = 0; w < 8; ++w) {
      const float p0 = __builtin_amdgcn_exp2f(__builtin_fmaf(st[2 * w], scale_log2e, neg_m));
      const float p1 = __builtin_amdgcn_exp2f(__builtin_fmaf(st[2 * w + 1], scale_log2e, neg_m));
      const uint32_t pk = pack2<T>(p0, p1);
      pf[w >> 2].w[w & 3] = pk;
      psum = add_pair<T>(pk, psum);
    }
    l_run += psum;
#pragma unroll
    for (int kk = 0; kk < 2; ++kk)
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        const Chunk16 vf = *reinterpret_cast<const Chunk16*>(vt + t * 32 * 128 + k_off[2 * sub + kk]);
        ot[t] = mma16<T>(vf, pf[kk], ot[t]);
      }
  }
}

// Normalise a wavefront's 32 x 64 output block and write it: ot[t][e] = O[query lrow][d = 32t + 8*(e/4) + 4*lhalf + e%4].
// The block is staged in LDS (stage_base: the workgroup's LDS, free by now; 32 x (64 + 8) elements per wavefront) so
// that it leaves as 128-byte rows.  out_head: first element of the head's columns in row 0 of this sequence.
template <typename T>
__device__ __forceinline__ void store_context(char* stage_base, int wave, int lane, const floatx16 (&ot)[2], float l_run,
                                              T* out_head, int row_pitch, int q0, int q_end) {
  const int lrow = lane & 31, lhalf = lane >> 5;
  const float l_tot = l_run + __shfl_xor(l_run, 32, kWave);
  const float inv = 1.0f / l_tot;
  T* stage_o = reinterpret_cast<T*>(stage_base) + wave * (32 * (kD + 8));
#pragma unroll
  for (int t = 0; t < 2; ++t)
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      Chunk8 c;
      c.w[0] = pack2<T>(ot[t][4 * g] * inv, ot[t][4 * g + 1] * inv);
      c.w[1] = pack2<T>(ot[t][4 * g + 2] * inv, ot[t][4 * g + 3] * inv);
      *reinterpret_cast<Chunk8*>(stage_o + lrow * (kD + 8) + t * 32 + 8 * g + 4 * lhalf) = c;
    }
#pragma unroll
  for (int p = 0; p < 4; ++p) {
    const int r = p * 8 + (lane >> 3), cchunk = lane & 7;
    const int qi = q0 + r;
    if (qi < q_end) {
      const Chunk16 x = *reinterpret_cast<const Chunk16*>(stage_o + r * (kD + 8) + cchunk * 8);
      *reinterpret_cast<Chunk16*>(out_head + (int64_t)qi * row_pitch + cchunk * 8) = x;
    }
  }
}

template <typename T, bool PACKED, bool VT, int NW>
__global__ __launch_bounds__(NW * 64, 16 / NW) void fused_attention_kernel(const T* __restrict__ q, const T* __restrict__ k,
                                                                 const T* __restrict__ v, const float* __restrict__ mask,
                                                                 T* __restrict__ out, const int32_t* __restrict__ cu,
                                                                 int heads, int seq, int v_pitch, float scale_log2e,
                                                                 float inv_scale) {
  // one LDS block: [2 x K tile | 2 x V^T tile | 2 x mask]; the front is reused for the output tile
  static_assert(NW == 4 || NW == 8, "four or eight wavefronts");
  constexpr int kBQ = NW * 32;    // queries per workgroup
  constexpr int kPieces = 8 / NW;  // 16-byte pieces of a K (V^T) tile per thread: the tile has 64 rows of 8
  constexpr int kKBytes = kBKV * 128, kVtBytes = kD * 128;
  constexpr int kTileBytes = 2 * kKBytes + 2 * kVtBytes + 2 * kBKV * 4, kOutBytes = NW * 32 * (kD + 8) * (int)sizeof(T);
  __shared__ __align__(16) char smem[kTileBytes > kOutBytes ? kTileBytes : kOutBytes];
  auto k_lds = [&](int stage) { return smem + stage * kKBytes; };
  auto vt_lds = [&](int stage) { return smem + 2 * kKBytes + stage * kVtBytes; };
  // additive mask per key, already divided by the score scale: it seeds the score accumulators
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
  const T* vb = v + (int64_t)bh * kD * (VT ? v_pitch : seq);

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

  // K/V tiles are register-staged: the global loads of tile t+1 are issued before the MFMAs of
  // tile t and written to the other LDS stage afterwards, so their latency hides behind compute.
  // Loads past the last key are clamped to valid memory: such keys carry a -1e30 mask, so a
  // duplicated K row is harmless; V^T columns past the last key may be uninitialised memory and
  // are zeroed on the way to LDS (0 * NaN would poison the output).
  // (Named vector registers, not arrays: an array captured by the two lambdas ends up in scratch.)
  u32x4 kreg0{}, kreg1{}, vreg0{}, vreg1{};
  float mreg = 0.f;
  auto load_regs = [&](int tile) {
    const int key0 = tile * kBKV;
    const int ch = tid & 7, r0 = tid >> 3;  // chunk and row of this lane's first 16-byte piece; second (four wavefronts): row + 32
    {
      const T* p0 = kb + (int64_t)min(key0 + r0, kv_len - 1) * kD + ch * 8;  // 128-byte K rows, coalesced
      kreg0 = *reinterpret_cast<const u32x4*>(p0);
      if (kPieces == 2) {
        const T* p1 = kb + (int64_t)min(key0 + r0 + 32, kv_len - 1) * kD + ch * 8;
        kreg1 = *reinterpret_cast<const u32x4*>(p1);
      }
    }
    if (VT) {
      const int ks = min(key0 + ch * 8, v_pitch - 8);
      vreg0 = *reinterpret_cast<const u32x4*>(vb + (int64_t)r0 * v_pitch + ks);
      if (kPieces == 2) vreg1 = *reinterpret_cast<const u32x4*>(vb + (int64_t)(r0 + 32) * v_pitch + ks);
    } else {
      const int key = min(key0 + (tid & 63), kv_len - 1), dch = tid >> 6;
      vreg0 = *reinterpret_cast<const u32x4*>(vb + (int64_t)key * kD + dch * 8);
      if (kPieces == 2) vreg1 = *reinterpret_cast<const u32x4*>(vb + (int64_t)key * kD + (dch + 4) * 8);
    }
    if (tid < kBKV) {
      const int key = key0 + tid;
      const float mv = mask ? mask[(int64_t)b * seq + min(key, kv_len - 1)] * inv_scale : 0.f;
      mreg = key < kv_len ? mv : kNegBig;
    }
  };
  auto put_vt = [&](u32x4 x, int tile, int stage, int drow, int ch) {
    if (tile * kBKV + kBKV > kv_len) {  // only the last tile: zero the keys past the end
      const int nv = kv_len - (tile * kBKV + ch * 8);  // valid keys in this chunk
#pragma unroll
      for (int w = 0; w < 4; ++w) {
        if (2 * w >= nv) x[w] = 0u;
        else if (2 * w + 1 >= nv) x[w] &= 0xffffu;
      }
    }
    // keys 8ch..8ch+3 and 8ch+4..8ch+7 go to the two 16-byte slots of their 16-key group
    char* row = vt_lds(stage) + drow * 128 + (ch & 1) * 8;
    const int slot = (ch >> 1) * 2, sw = (drow >> 1) & 7;
    *reinterpret_cast<u32x2*>(row + ((slot ^ sw) << 4)) = u32x2{x[0], x[1]};
    *reinterpret_cast<u32x2*>(row + (((slot + 1) ^ sw) << 4)) = u32x2{x[2], x[3]};
  };
  auto scatter_v = [&](u32x4 x, int stage, int dch) {
    const int key = tid & 63;
    const int pos = vt_pos(key & 15), slot = (key >> 4) * 2 + (pos >> 3);
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int drow = dch * 8 + j;
      const uint32_t word = x[j >> 1];
      *reinterpret_cast<uint16_t*>(vt_lds(stage) + drow * 128 + ((slot ^ ((drow >> 1) & 7)) << 4) + (pos & 7) * 2) =
          (uint16_t)((j & 1) ? (word >> 16) : (word & 0xffffu));
    }
  };
  auto store_tile_lds = [&](int tile, int stage) {
    const int ch = tid & 7, r0 = tid >> 3;
    *reinterpret_cast<u32x4*>(k_lds(stage) + r0 * 128 + ((ch ^ ((r0 >> 1) & 7)) << 4)) = kreg0;
    if (kPieces == 2) *reinterpret_cast<u32x4*>(k_lds(stage) + (r0 + 32) * 128 + ((ch ^ ((r0 >> 1) & 7)) << 4)) = kreg1;  // +32 keeps the swizzle
    if (VT) {
      put_vt(vreg0, tile, stage, r0, ch);
      if (kPieces == 2) put_vt(vreg1, tile, stage, r0 + 32, ch);
    } else {
      scatter_v(vreg0, stage, tid >> 6);
      if (kPieces == 2) scatter_v(vreg1, stage, (tid >> 6) + 4);
    }
    if (tid < kBKV) mask_lds(stage)[tid] = mreg;
  };

  // One 64-key tile from LDS stage STAGE (a compile-time constant so every LDS address is a
  // per-lane base plus an immediate).
  const int k_lane = lrow * 128, k_sw = (lrow >> 1) & 7;
  int k_off[4];
#pragma unroll
  for (int kk = 0; kk < 4; ++kk) k_off[kk] = k_lane + (((2 * kk + lhalf) ^ k_sw) << 4);  // rows +32 keep the swizzle
  auto compute_tile = [&](auto stage_c) {
    constexpr int STAGE = decltype(stage_c)::value;
    attention_tile<T>(smem + STAGE * kKBytes, smem + 2 * kKBytes + STAGE * kVtBytes,
                      reinterpret_cast<const float*>(smem + 2 * kKBytes + 2 * kVtBytes) + STAGE * kBKV, qf, k_off, lhalf,
                      scale_log2e, ot, m_run, l_run);
  };

  const int tiles = (kv_len + kBKV - 1) / kBKV;
  const bool wave_active = q0 < q_len;
  load_regs(0);
  store_tile_lds(0, 0);
  __syncthreads();
  for (int tile = 0; tile < tiles; tile += 2) {
    if (tile + 1 < tiles) load_regs(tile + 1);
    if (wave_active) compute_tile(std::integral_constant<int, 0>{});
    if (tile + 1 < tiles) store_tile_lds(tile + 1, 1);
    __syncthreads();
    if (tile + 1 >= tiles) break;
    if (tile + 2 < tiles) load_regs(tile + 2);
    if (wave_active) compute_tile(std::integral_constant<int, 1>{});
    if (tile + 2 < tiles) store_tile_lds(tile + 2, 0);
    __syncthreads();
  }

  store_context<T>(smem, wave, lane, ot, l_run, out + (int64_t)out_row0 * (heads * kD) + head * kD, heads * kD, q0,
                   min(q_len, seq));
}

}  // namespace ttmi

namespace ttmi {
// attention_f32.hip: the fp32 form
int fused_attention_f32(const float* q, const float* k, const float* v, const float* mask, float* out, const int32_t* cu,
                        int64_t batch, int64_t heads, int64_t seq, int64_t v_seq_pitch, float scale, int nw, float* absmax,
                        hipStream_t s);

// absmax / slots_written: see ttmi_fused_attention_absmax; both null for the plain entry point
static int fused_attention_impl(const void* q, const void* k, const void* v, const float* mask, void* out,
                                const int32_t* cu_seqlens, int64_t batch, int64_t heads, int64_t seq, int64_t head_dim,
                                int64_t v_seq_pitch, float scale, int dtype, float* absmax, int* slots_written, void* stream) {
  TTMI_REQUIRE(q && k && v && out, "null tensor");
  TTMI_REQUIRE(head_dim == kD, "fused attention is built for head_dim 64");
  TTMI_REQUIRE(dtype == TTMI_F16 || dtype == TTMI_BF16 || dtype == TTMI_F32, "fused attention is built for fp16 / bf16 / fp32");
  TTMI_REQUIRE(batch > 0 && heads > 0 && seq > 0 && batch * heads < 65536 && seq < (1 << 24), "bad shape");
  TTMI_REQUIRE(v_seq_pitch == 0 || (v_seq_pitch >= seq && v_seq_pitch % 8 == 0 && v_seq_pitch < (1 << 24)),
               "v_seq_pitch must be 0 or a multiple of 8 that is >= seq");
  TTMI_REQUIRE(scale > 0.f, "scale must be positive");
  uintptr_t bits = reinterpret_cast<uintptr_t>(q) | reinterpret_cast<uintptr_t>(k) | reinterpret_cast<uintptr_t>(v) |
                   reinterpret_cast<uintptr_t>(out);
  TTMI_REQUIRE((bits & 15) == 0, "tensors must be 16-byte aligned");
  // Eight wavefronts (256 queries) per workgroup stream the keys and values of their head once for twice the queries:
  // a workgroup of that size costs about 1.6 times one of four wavefronts (20 x 136 tokens: 7.4 against 9.2 us;
  // 64 x 512: 77 against 81).  Four win where the sequence fits them (up to 128 tokens), where two blocks of 256
  // queries stand against three of 128 (257..384 tokens; 64 x 300: 44 against 49 us), and where even their workgroups
  // are fewer than the compute units (4 x 512 tokens: 12.4 against 13.7 us).
  static const int cus = [] {
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0)
      n = 256;
    return n;
  }();
  const bool fits_four = seq <= 128 || 8 * ceil_div(seq, 256) >= 5 * ceil_div(seq, 128);
  int nw = (fits_four || ceil_div(seq, 128) * batch * heads < (int64_t)cus) ? 4 : 8;
  // TTMI_ATTENTION_WAVES=4 / 8 overrides the choice (A/B timing, and tests of the eight-wavefront form on small shapes)
  const int force = kernel_switch(kSwitchAttentionWaves);
  if (force == 4 || force == 8) nw = force;
  const dim3 grid((unsigned)ceil_div(seq, nw * 32), (unsigned)(batch * heads));
  const float sl2 = scale * 1.4426950408889634f, inv_scale = 1.0f / scale;
  hipStream_t s = (hipStream_t)stream;
  if (dtype == TTMI_F32) {
    // the per-workgroup maxima: dense fp32 batches whose workgroups fit the slots
    const bool leave_maxima = absmax != nullptr && cu_seqlens == nullptr && (int64_t)grid.x * grid.y <= TTMI_ABSMAX_SLOTS;
    const int rc = fused_attention_f32((const float*)q, (const float*)k, (const float*)v, mask, (float*)out, cu_seqlens, batch,
                                       heads, seq, v_seq_pitch, scale, nw, leave_maxima ? absmax : nullptr, s);
    if (rc == 0 && leave_maxima && slots_written != nullptr) *slots_written = TTMI_ABSMAX_SLOTS;
    return rc;
  }
#define TTMI_FA_LAUNCH(T, PACKED, VT, NW)                                                                              \
  hipLaunchKernelGGL((fused_attention_kernel<T, PACKED, VT, NW>), grid, dim3(NW * 64), 0, s, (const T*)q, (const T*)k, \
                     (const T*)v, mask, (T*)out, cu_seqlens, (int)heads, (int)seq, (int)v_seq_pitch, sl2, inv_scale)
#define TTMI_FA_WAVES(T, PACKED, VT)                  \
  do {                                                \
    if (nw == 8) TTMI_FA_LAUNCH(T, PACKED, VT, 8);    \
    else TTMI_FA_LAUNCH(T, PACKED, VT, 4);            \
  } while (0)
#define TTMI_FA_LAYOUT(T, PACKED)                    \
  do {                                               \
    if (v_seq_pitch) TTMI_FA_WAVES(T, PACKED, true); \
    else TTMI_FA_WAVES(T, PACKED, false);            \
  } while (0)
  if (dtype == TTMI_F16) {
    if (cu_seqlens) TTMI_FA_LAYOUT(f16, true); else TTMI_FA_LAYOUT(f16, false);
  } else {
    if (cu_seqlens) TTMI_FA_LAYOUT(bf16, true); else TTMI_FA_LAYOUT(bf16, false);
  }
#undef TTMI_FA_LAYOUT
#undef TTMI_FA_WAVES
#undef TTMI_FA_LAUNCH
  return launch_status("fused_attention");
}
}  // namespace ttmi

using namespace ttmi;

extern "C" {

int ttmi_fused_attention(const void* q, const void* k, const void* v, const float* mask, void* out,
                         const int32_t* cu_seqlens, int64_t batch, int64_t heads, int64_t seq, int64_t head_dim,
                         int64_t v_seq_pitch, float scale, int dtype, void* stream) {
  return fused_attention_impl(q, k, v, mask, out, cu_seqlens, batch, heads, seq, head_dim, v_seq_pitch, scale, dtype, nullptr,
                              nullptr, stream);
}

int ttmi_fused_attention_absmax(const void* q, const void* k, const void* v, const float* mask, void* out,
                                const int32_t* cu_seqlens, int64_t batch, int64_t heads, int64_t seq, int64_t head_dim,
                                int64_t v_seq_pitch, float scale, int dtype, float* absmax_slots, int* slots_written,
                                void* stream) {
  TTMI_REQUIRE(absmax_slots && slots_written, "null absmax arguments");
  *slots_written = 0;
  return fused_attention_impl(q, k, v, mask, out, cu_seqlens, batch, heads, seq, head_dim, v_seq_pitch, scale, dtype,
                              absmax_slots, slots_written, stream);
}

}  // extern "C"
