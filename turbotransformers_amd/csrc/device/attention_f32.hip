// Fused self-attention for head_dim 64 in fp32:  out = softmax(scale * Q K^T + mask) V  in one kernel, the fp32
// counterpart of attention.hip (which serves fp16 / bf16).  It replaces the batch_gemm3 -> ApplyMaskAndSoftmax ->
// batch_gemm4 -> TransposeForScore chain of layers/multi_headed_attention.cpp:323-354 when the caller does not ask for
// the probabilities: the [B,h,S,S] scores, written and read twice by that chain, never reach HBM.
//
// Same formulation as the 16-bit kernel, on v_mfma_f32_32x32x2_f32: scores are computed TRANSPOSED,
//     St[key, query] = K_tile[key, :] . Q[query, :]      (A = K from LDS, B = Q from registers)
// so a lane holds one query column and 16 key rows of a 32-key sub-tile; the online-softmax statistics are lane-local
// plus one exchange between the half-wavefronts.  A 32x32x2 instruction takes K index 0 from lanes 0-31 and K index 1
// from lanes 32-63, and which two indices of the long dimension a given instruction pairs is free as long as both
// operands agree.  Accumulator register 4g+i of a lane in half h is key 8g + 4h + i: pairing keys (8g+i, 8g+4+i)
// in instruction (g, i) makes the probabilities, still in the accumulator registers, the B operand of
//     Ot[d, query] += Vt[d, keys] . Pt[keys, query]      (A = V^T from LDS, B = P from registers)
// with A read as the 16-byte chunk (2g+h) of a V^T row: four keys, one per instruction.  The first product pairs the
// head dimension the same way (chunk 2kk+h of a K row and of a Q row).  Everything stays fp32; exp is exp2 with
// scale*log2(e) folded into the argument, the additive mask (divided by the scale) seeds the score accumulators, the
// running maximum is exact.  The matrix pipe bounds the kernel (4*S*64 FLOP per query and head at 157 TFLOP/s).
//
// V may be given transposed ([B,h,d,pitch], as the QKV epilogue writes it with v_seq_pitch: its tiles are then copied)
// or row-major ([B,h,S,d]: a thread scatters its four values of a key into four V^T rows).  With cu_seqlens q,k,v are
// the padded tensors of a packed batch (S = longest sequence): keys and queries past a sequence's length are never
// read and the output is packed [sum(len), h*64].
#include <cstdlib>
#include <mutex>
#include <set>

#include "common.h"

namespace ttmi {

namespace {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float floatx4 __attribute__((ext_vector_type(4), may_alias));

constexpr int kD = 64;           // head dim
constexpr int kBKV = 64;         // keys per LDS tile
constexpr int kRow = 256;        // bytes of a K row (64 floats) and of a V^T row (64 keys)
constexpr float kNegBig = -1.0e30f;

// four K indices of both operands, one per instruction
__device__ __forceinline__ floatx16 mma4(const floatx4& a, const floatx4& b, floatx16 c) {
#pragma unroll
  for (int j = 0; j < 4; ++j) c = __builtin_amdgcn_mfma_f32_32x32x2f32(a[j], b[j], c, 0, 0, 0);
  return c;
}

// 16-byte chunk `chunk` of row `row` of a tile with 256-byte rows: the 16 lanes the LDS serves together read one chunk
// column of 16 different rows, so the chunk index is XORed with the row
__device__ __forceinline__ int tile_off(int row, int chunk) { return row * kRow + ((chunk ^ (row & 15)) << 4); }

template <int NW>
constexpr int lds_bytes() {
  constexpr int tiles = 4 * kBKV * kRow + 2 * kBKV * 4, outb = NW * 32 * (kD + 4) * 4;
  return tiles > outb ? tiles : outb;
}

template <int NW, bool VT, bool PACKED>
__global__ __launch_bounds__(NW * 64) __attribute__((amdgpu_waves_per_eu(2))) void fused_attention_f32_kernel(
    const float* __restrict__ q, const float* __restrict__ k, const float* __restrict__ v, const float* __restrict__ mask,
    float* __restrict__ out, const int32_t* __restrict__ cu, int heads, int seq, int v_pitch, float scale_log2e,
    float inv_scale, float* __restrict__ absmax) {
  static_assert(NW == 4 || NW == 8, "four or eight wavefronts");
  constexpr int kBQ = NW * 32;               // queries per workgroup
  constexpr int kPieces = 1024 / (NW * 64);  // 16-byte pieces of a K (V^T) tile per thread: 64 rows of 16
  constexpr int kTile = kBKV * kRow;         // 16 KB
  // dynamic LDS (lds_bytes<NW>(), more than the 64 KB a kernel gets without asking):
  // [2 x K tile | 2 x V^T tile | 2 x mask]; the front is reused for the output tile
  extern __shared__ __align__(16) char smem[];

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

  const float* qb = q + (int64_t)bh * seq * kD;
  const float* kb = k + (int64_t)bh * seq * kD;
  const float* vb = v + (int64_t)bh * kD * (VT ? v_pitch : seq);

  // Q fragments: B operand of the first product, chunk 2kk+lhalf of the lane's query row
  floatx4 qf[8];
  {
    const int qi = q0 + lrow;
#pragma unroll
    for (int kk = 0; kk < 8; ++kk) {
      if (qi < q_len) qf[kk] = *reinterpret_cast<const floatx4*>(qb + (int64_t)qi * kD + (2 * kk + lhalf) * 4);
      else qf[kk] = floatx4{0.f, 0.f, 0.f, 0.f};
    }
  }

  floatx16 ot[2];
#pragma unroll
  for (int t = 0; t < 2; ++t)
#pragma unroll
    for (int e = 0; e < 16; ++e) ot[t][e] = 0.f;
  float m_run = kNegBig, l_run = 0.f;

  // tile staging: thread -> (row r0 + 64*NW/16*p, chunk ch); global -> registers one tile ahead -> LDS
  constexpr int kRowsPerPass = NW * 64 / 16;
  const int ch = tid & 15, r0 = tid >> 4;
  floatx4 kreg[kPieces], vreg[kPieces];
  float mreg = 0.f;

#define TTMI_FA32_LOAD(tile_)                                                                                      \
  do {                                                                                                              \
    const int key0_ = (tile_) * kBKV;                                                                               \
    _Pragma("unroll") for (int p = 0; p < kPieces; ++p) {                                                           \
      const int r_ = r0 + p * kRowsPerPass;                                                                         \
      kreg[p] = *reinterpret_cast<const floatx4*>(kb + (int64_t)min(key0_ + r_, kv_len - 1) * kD + ch * 4);         \
      if (VT) { /* row r_ of V^T, keys 4ch.. of the tile */                                                         \
        const int ks_ = min(key0_ + ch * 4, v_pitch - 4);                                                           \
        vreg[p] = *reinterpret_cast<const floatx4*>(vb + (int64_t)r_ * v_pitch + ks_);                              \
      } else { /* key r_ of the tile, head dimensions 4ch.. */                                                      \
        vreg[p] = *reinterpret_cast<const floatx4*>(vb + (int64_t)min(key0_ + r_, kv_len - 1) * kD + ch * 4);       \
      }                                                                                                             \
    }                                                                                                               \
    if (tid < kBKV) {                                                                                               \
      const int key_ = key0_ + tid;                                                                                 \
      const float mv_ = mask ? mask[(int64_t)b * seq + min(key_, kv_len - 1)] * inv_scale : 0.f;                    \
      mreg = key_ < kv_len ? mv_ : kNegBig;                                                                         \
    }                                                                                                               \
  } while (0)

#define TTMI_FA32_STORE(tile_, stage_)                                                                             \
  do {                                                                                                              \
    char* const kt_ = smem + (stage_) * kTile;                                                                      \
    char* const vt_ = smem + 2 * kTile + (stage_) * kTile;                                                          \
    const int nv_ = kv_len - ((tile_) * kBKV + ch * 4); /* valid keys in this thread's V^T chunk */                 \
    _Pragma("unroll") for (int p = 0; p < kPieces; ++p) {                                                           \
      const int r_ = r0 + p * kRowsPerPass;                                                                         \
      *reinterpret_cast<floatx4*>(kt_ + tile_off(r_, ch)) = kreg[p];                                                \
      floatx4 x_ = vreg[p];                                                                                         \
      if (VT) {                                                                                                     \
        if (nv_ < 4) { /* only in the last tile: keys past the end may hold anything, zero them */                  \
          _Pragma("unroll") for (int w = 0; w < 4; ++w) if (w >= nv_) x_[w] = 0.f;                                  \
        }                                                                                                           \
        *reinterpret_cast<floatx4*>(vt_ + tile_off(r_, ch)) = x_;                                                   \
      } else { /* V^T[d = 4ch + w][key r_]: float r_ % 4 of chunk r_ / 4 of row d; keys past the end are zero */    \
        const bool live_ = (tile_) * kBKV + r_ < kv_len;                                                            \
        _Pragma("unroll") for (int w = 0; w < 4; ++w)                                                               \
          *reinterpret_cast<float*>(vt_ + tile_off(ch * 4 + w, r_ >> 2) + (r_ & 3) * 4) = live_ ? x_[w] : 0.f;      \
      }                                                                                                             \
    }                                                                                                               \
    if (tid < kBKV) reinterpret_cast<float*>(smem + 4 * kTile)[(stage_) * kBKV + tid] = mreg;                       \
  } while (0)

  // One 64-key tile from LDS stage STAGE.  m_run is kept in raw score units; p = exp2(s*c - m*c), c = scale*log2(e).
  auto compute_tile = [&](auto stage_c) {
    constexpr int STAGE = decltype(stage_c)::value;
    const char* kt = smem + STAGE * kTile;
    const char* vt = smem + 2 * kTile + STAGE * kTile;
    const float* mk = reinterpret_cast<const float*>(smem + 4 * kTile) + STAGE * kBKV;
#pragma unroll
    for (int sub = 0; sub < 2; ++sub) {  // two 32-key sub-tiles
      const int sk = sub * 32;
      // st[4g+i] = score of (key sk + 8g + 4*lhalf + i, query lrow), seeded with mask/scale
      floatx16 st;
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const float4 mv = *reinterpret_cast<const float4*>(mk + sk + 8 * g + 4 * lhalf);
        st[4 * g] = mv.x, st[4 * g + 1] = mv.y, st[4 * g + 2] = mv.z, st[4 * g + 3] = mv.w;
      }
#pragma unroll
      for (int kk = 0; kk < 8; ++kk) {
        const floatx4 kf = *reinterpret_cast<const floatx4*>(kt + tile_off(sk + lrow, 2 * kk + lhalf));
        st = mma4(kf, qf[kk], st);
      }
      float mx = st[0];
#pragma unroll
      for (int e = 1; e < 16; ++e) mx = fmaxf(mx, st[e]);
      {
        // the other half-wavefront holds the remaining 16 keys of this query
        const auto sw = __builtin_amdgcn_permlane32_swap(__builtin_bit_cast(unsigned, mx), __builtin_bit_cast(unsigned, mx), false, false);
        mx = fmaxf(__builtin_bit_cast(float, sw[0]), __builtin_bit_cast(float, sw[1]));
      }
      if (__any(mx > m_run)) {
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
      float psum = 0.f;
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        st[e] = __builtin_amdgcn_exp2f(__builtin_fmaf(st[e], scale_log2e, neg_m));
        psum += st[e];
      }
      l_run += psum;
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const floatx4 pf{st[4 * g], st[4 * g + 1], st[4 * g + 2], st[4 * g + 3]};
#pragma unroll
        for (int t = 0; t < 2; ++t) {
          const floatx4 vf = *reinterpret_cast<const floatx4*>(vt + tile_off(t * 32 + lrow, sk / 4 + 2 * g + lhalf));
          ot[t] = mma4(vf, pf, ot[t]);
        }
      }
    }
  };

  const int tiles = (kv_len + kBKV - 1) / kBKV;
  const bool wave_active = q0 < q_len;
  TTMI_FA32_LOAD(0);
  TTMI_FA32_STORE(0, 0);
  __syncthreads();
  for (int tile = 0; tile < tiles; tile += 2) {
    if (tile + 1 < tiles) TTMI_FA32_LOAD(tile + 1);
    if (wave_active) compute_tile(std::integral_constant<int, 0>{});
    if (tile + 1 < tiles) TTMI_FA32_STORE(tile + 1, 1);
    __syncthreads();
    if (tile + 1 >= tiles) break;
    if (tile + 2 < tiles) TTMI_FA32_LOAD(tile + 2);
    if (wave_active) compute_tile(std::integral_constant<int, 1>{});
    if (tile + 2 < tiles) TTMI_FA32_STORE(tile + 2, 0);
    __syncthreads();
  }
#undef TTMI_FA32_LOAD
#undef TTMI_FA32_STORE

  // normalise and write: ot[t][4g+i] = O[query lrow][d = 32t + 8g + 4*lhalf + i]
  const float l_tot = l_run + __shfl_xor(l_run, 32, kWave);
  const float inv = 1.0f / l_tot;
  // stage the wavefront's 32 x 64 tile in LDS (every wavefront is past the last tile barrier) to store 256-byte rows
  float* stage_o = reinterpret_cast<float*>(smem) + wave * (32 * (kD + 4));
#pragma unroll
  for (int t = 0; t < 2; ++t)
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const floatx4 c{ot[t][4 * g] * inv, ot[t][4 * g + 1] * inv, ot[t][4 * g + 2] * inv, ot[t][4 * g + 3] * inv};
      *reinterpret_cast<floatx4*>(stage_o + lrow * (kD + 4) + t * 32 + 8 * g + 4 * lhalf) = c;
    }
  const int hd = heads * kD;
  float amax = 0.f;
#pragma unroll
  for (int p = 0; p < 8; ++p) {
    const int r = p * 4 + (lane >> 4), cchunk = lane & 15;
    const int qi = q0 + r;
    if (qi < q_len) {
      const floatx4 x = *reinterpret_cast<const floatx4*>(stage_o + r * (kD + 4) + cchunk * 4);
      *reinterpret_cast<floatx4*>(out + ((int64_t)out_row0 + qi) * hd + head * kD + cchunk * 4) = x;
      amax = fmaxf(fmaxf(amax, fmaxf(fabsf(x[0]), fabsf(x[1]))), fmaxf(fabsf(x[2]), fabsf(x[3])));
    }
  }
  // Optional (dense batches): max|out| of this workgroup to its slot, for the int8 Linear that quantises `out` next;
  // workgroup 0 zeroes the slots no workgroup owns, so every slot is written by every launch.
  if (absmax != nullptr) {
    amax = group_max<kWave>(amax);
    __syncthreads();  // every wavefront is done with its share of the output stage
    float* red = reinterpret_cast<float*>(smem);
    if (lane == 0) red[wave] = amax;
    __syncthreads();
    const int wg = (int)(blockIdx.y * gridDim.x + blockIdx.x), wgs = (int)(gridDim.x * gridDim.y);
    if (tid == 0) {
      float m = red[0];
#pragma unroll
      for (int w = 1; w < NW; ++w) m = fmaxf(m, red[w]);
      absmax[wg] = m;
    }
    if (wg == 0)
      for (int i = wgs + tid; i < TTMI_ABSMAX_SLOTS; i += NW * 64) absmax[i] = 0.f;
  }
}

}  // namespace

// Launch; arguments were checked by ttmi_fused_attention.
int fused_attention_f32(const float* q, const float* k, const float* v, const float* mask, float* out, const int32_t* cu,
                        int64_t batch, int64_t heads, int64_t seq, int64_t v_seq_pitch, float scale, int nw, float* absmax,
                        hipStream_t s) {
  const dim3 grid((unsigned)ceil_div(seq, nw * 32), (unsigned)(batch * heads));
  const float sl2 = scale * 1.4426950408889634f, inv_scale = 1.0f / scale;
  // more than 64 KB of dynamic LDS: the limit is raised once per kernel and device
  auto launch = [&](auto kern, int threads, int lds) -> int {
    static std::mutex mu;
    static std::set<std::pair<const void*, int>> done;
    int dev = 0;
    TTMI_HIP(hipGetDevice(&dev));
    {
      std::lock_guard<std::mutex> lock(mu);
      const void* fn = reinterpret_cast<const void*>(kern);
      if (done.count({fn, dev}) == 0) {
        TTMI_HIP(hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, lds));
        done.insert({fn, dev});
      }
    }
    hipLaunchKernelGGL(kern, grid, dim3(threads), lds, s, q, k, v, mask, out, cu, (int)heads, (int)seq, (int)v_seq_pitch, sl2,
                       inv_scale, absmax);
    return 0;
  };
  const bool vt = v_seq_pitch > 0, packed = cu != nullptr;
  int rc = 0;
#define TTMI_FA32_CASE(NW, VT, PACKED) rc = launch(&fused_attention_f32_kernel<NW, VT, PACKED>, NW * 64, lds_bytes<NW>())
  if (nw == 8) {
    if (vt) { if (packed) TTMI_FA32_CASE(8, true, true); else TTMI_FA32_CASE(8, true, false); }
    else { if (packed) TTMI_FA32_CASE(8, false, true); else TTMI_FA32_CASE(8, false, false); }
  } else {
    if (vt) { if (packed) TTMI_FA32_CASE(4, true, true); else TTMI_FA32_CASE(4, true, false); }
    else { if (packed) TTMI_FA32_CASE(4, false, true); else TTMI_FA32_CASE(4, false, false); }
  }
#undef TTMI_FA32_CASE
  if (rc != 0) return rc;
  return launch_status("fused_attention_f32_kernel");
}

}  // namespace ttmi
