// TEST INFRASTRUCTURE -- not part of the product.
//
// CPU restatement of the CPU branch of TurboTransformers' BERT encoder-layer hot path, in
// plain C++17 + OpenMP behind a C ABI (loaded with ctypes by tests/, by the smoke check and
// by bench.py's cpu_baseline leg only).  Every function cites the reference file:line it
// follows (paths relative to the reference tree, turbo_transformers/...).  The reference
// itself cannot be built offline (empty submodules, network fetches), so this file restates
// its algorithms; tests/test_oracle_*.py pin each function against independent checks
// (library routines, closed forms, brute force, HuggingFace BERT goldens).
//
// GEMMs go through cblas_sgemm of whichever BLAS oracle_load_blas() finds (the reference's
// provider is MKL or OpenBLAS); without one a blocked in-file sgemm is used.
#include <dlfcn.h>
#include <omp.h>

#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <limits>
#include <numeric>
#include <string>
#include <vector>

#define ORACLE_API extern "C" __attribute__((visibility("default")))

namespace {

// ------------------------------------------------------------------ BLAS plumbing -------
enum { RowMajor = 101, NoTrans = 111, Trans = 112 };
typedef void (*sgemm32_t)(int, int, int, int, int, int, float, const float*, int, const float*, int, float,
                          float*, int);
typedef void (*sgemm64_t)(int, int, int, int64_t, int64_t, int64_t, float, const float*, int64_t, const float*,
                          int64_t, float, float*, int64_t);
sgemm32_t g_sgemm32 = nullptr;
sgemm64_t g_sgemm64 = nullptr;
std::string g_blas_name = "builtin-blocked-sgemm (no vendor BLAS)";
void (*g_set_threads)(int) = nullptr;

// C[M,N] = alpha * op(A) * op(B) + beta * C, row-major; only A non-transposed is needed here.
void builtin_sgemm(bool trans_b, int64_t M, int64_t N, int64_t K, float alpha, const float* A, int64_t lda,
                   const float* B, int64_t ldb, float beta, float* C, int64_t ldc) {
  constexpr int64_t TM = 64, TN = 256, TK = 256;
#pragma omp parallel for collapse(2) schedule(static)
  for (int64_t m0 = 0; m0 < M; m0 += TM) {
    for (int64_t n0 = 0; n0 < N; n0 += TN) {
      const int64_t m1 = std::min(M, m0 + TM), n1 = std::min(N, n0 + TN);
      std::vector<float> acc((m1 - m0) * (n1 - n0), 0.f);
      const int64_t w = n1 - n0;
      for (int64_t k0 = 0; k0 < K; k0 += TK) {
        const int64_t k1 = std::min(K, k0 + TK);
        for (int64_t m = m0; m < m1; ++m) {
          float* arow = acc.data() + (m - m0) * w;
          if (!trans_b) {
            for (int64_t k = k0; k < k1; ++k) {
              const float a = A[m * lda + k];
              const float* brow = B + k * ldb + n0;
#pragma omp simd
              for (int64_t n = 0; n < w; ++n) arow[n] += a * brow[n];
            }
          } else {
            for (int64_t n = n0; n < n1; ++n) {
              const float* brow = B + n * ldb;
              float s = 0.f;
#pragma omp simd reduction(+ : s)
              for (int64_t k = k0; k < k1; ++k) s += A[m * lda + k] * brow[k];
              arow[n - n0] += s;
            }
          }
        }
      }
      for (int64_t m = m0; m < m1; ++m)
        for (int64_t n = n0; n < n1; ++n) {
          float& c = C[m * ldc + n];
          c = alpha * acc[(m - m0) * w + (n - n0)] + (beta == 0.f ? 0.f : beta * c);
        }
    }
  }
}

void sgemm(bool trans_b, int64_t M, int64_t N, int64_t K, float alpha, const float* A, int64_t lda,
           const float* B, int64_t ldb, float beta, float* C, int64_t ldc) {
  if (M == 0 || N == 0) return;
  if (g_sgemm64) {
    g_sgemm64(RowMajor, NoTrans, trans_b ? Trans : NoTrans, M, N, K, alpha, A, lda, B, ldb, beta, C, ldc);
  } else if (g_sgemm32) {
    g_sgemm32(RowMajor, NoTrans, trans_b ? Trans : NoTrans, (int)M, (int)N, (int)K, alpha, A, (int)lda, B, (int)ldb,
              beta, C, (int)ldc);
  } else {
    builtin_sgemm(trans_b, M, N, K, alpha, A, lda, B, ldb, beta, C, ldc);
  }
}

}  // namespace

// Try to bind cblas_sgemm from `path`.  kind: 0 = LP64 symbols (cblas_sgemm: MKL, system
// OpenBLAS), 1 = the ILP64 OpenBLAS bundled in the NumPy/SciPy wheels (scipy_cblas_sgemm64_).
ORACLE_API int oracle_load_blas(const char* path, int kind) {
  void* h = dlopen(path, RTLD_NOW | RTLD_LOCAL);
  if (!h) return -1;
  if (kind == 0) {
    auto f = (sgemm32_t)dlsym(h, "cblas_sgemm");
    if (!f) return -2;
    g_sgemm32 = f;
    g_sgemm64 = nullptr;
    g_set_threads = (void (*)(int))dlsym(h, "MKL_Set_Num_Threads");
    if (!g_set_threads) g_set_threads = (void (*)(int))dlsym(h, "openblas_set_num_threads");
  } else {
    auto f = (sgemm64_t)dlsym(h, "scipy_cblas_sgemm64_");
    if (!f) f = (sgemm64_t)dlsym(h, "cblas_sgemm64_");
    if (!f) return -2;
    g_sgemm64 = f;
    g_sgemm32 = nullptr;
    g_set_threads = (void (*)(int))dlsym(h, "scipy_openblas_set_num_threads64_");
    if (!g_set_threads) g_set_threads = (void (*)(int))dlsym(h, "openblas_set_num_threads64_");
  }
  g_blas_name = path;
  return 0;
}
ORACLE_API void oracle_use_builtin_blas() {
  g_sgemm32 = nullptr;
  g_sgemm64 = nullptr;
  g_set_threads = nullptr;
  g_blas_name = "builtin-blocked-sgemm (no vendor BLAS)";
}
ORACLE_API const char* oracle_blas_name() { return g_blas_name.c_str(); }
// core::SetNumThreads (core/config.cpp:23-34): BLAS threads + OpenMP threads.
ORACLE_API void oracle_set_num_threads(int n) {
  omp_set_num_threads(n);
  if (g_set_threads) g_set_threads(n);
}
ORACLE_API int oracle_max_threads() { return omp_get_max_threads(); }

// ------------------------------------------------------------------------ kernels -------

// kernels::MatMul, CPU branch (layers/kernels/mat_mul.cpp:37-64): row-major
// C[M,N] = alpha * A[M,K] * (b_trans ? B[N,K]^T : B[K,N]) + beta * C, lda=K, ldb = b_trans?K:N, ldc=N.
ORACLE_API void oracle_matmul(const float* A, const float* B, float* C, int64_t M, int64_t N, int64_t K,
                              int b_trans, float alpha, float beta) {
  sgemm(b_trans != 0, M, N, K, alpha, A, K, B, b_trans ? K : N, beta, C, N);
}

// kernels::BatchMatMul, CPU branch (layers/kernels/mat_mul.cpp:126-190): `batch` independent
// problems at offsets M*K, (K*N), M*N; cblas_sgemm_batch == a loop of cblas_sgemm
// (core/blas_openblas.cpp:20-41).
ORACLE_API void oracle_batch_matmul(const float* A, const float* B, float* C, int64_t batch, int64_t M,
                                    int64_t N, int64_t K, int b_trans, float alpha, float beta) {
  for (int64_t i = 0; i < batch; ++i)
    sgemm(b_trans != 0, M, N, K, alpha, A + i * M * K, K, B + i * K * N, b_trans ? K : N, beta, C + i * M * N, N);
}

// kernels::SplitAddBiasTransposeForScore, 3 outputs (layers/kernels/transpose.cpp:347-390):
// in[B,S,3,h,d] + bias[3,h,d] -> q,k,v[B,h,S,d].
ORACLE_API void oracle_split_add_bias_transpose(const float* in, const float* bias, float* q, float* k, float* v,
                                                int64_t B, int64_t S, int64_t h, int64_t d) {
#pragma omp parallel for
  for (int64_t idx = 0; idx < B * 3 * S; ++idx) {
    const int64_t b = idx / (S * 3), s = idx / 3 % S, w = idx % 3;
    float* out = w == 0 ? q : (w == 1 ? k : v);
    for (int64_t head = 0; head < h; ++head) {
      const float* src = in + (b * S + s) * 3 * h * d + w * h * d + head * d;
      const float* bp = bias + w * h * d + head * d;
      float* dst = out + ((b * h + head) * S + s) * d;
      for (int64_t i = 0; i < d; ++i) dst[i] = src[i] + bp[i];
    }
  }
}

// kernels::SplitAddBiasTransposeForScorePad (layers/kernels/transpose.cpp:501-564): packed
// in[sum(len),3,h,d] -> zero-initialised q,k,v[B,h,maxS,d]; rows >= len[b] stay 0 (no bias).
ORACLE_API void oracle_split_add_bias_transpose_pad(const float* in, const float* bias, float* q, float* k,
                                                    float* v, const int64_t* lens, int64_t B, int64_t maxS,
                                                    int64_t h, int64_t d) {
  const size_t bytes = (size_t)(B * maxS * h * d) * sizeof(float);
  std::memset(q, 0, bytes);
  std::memset(k, 0, bytes);
  std::memset(v, 0, bytes);
#pragma omp parallel for
  for (int64_t idx = 0; idx < B * 3 * maxS; ++idx) {
    const int64_t b = idx / (maxS * 3), s = idx / 3 % maxS, w = idx % 3;
    if (s >= lens[b]) continue;
    const int64_t acc = std::accumulate(lens, lens + b, (int64_t)0);
    float* out = w == 0 ? q : (w == 1 ? k : v);
    for (int64_t head = 0; head < h; ++head) {
      const float* src = in + (acc + s) * 3 * h * d + w * h * d + head * d;
      const float* bp = bias + w * h * d + head * d;
      float* dst = out + ((b * h + head) * maxS + s) * d;
      for (int64_t i = 0; i < d; ++i) dst[i] = src[i] + bp[i];
    }
  }
}

// kernels::TransposeForScore (layers/kernels/transpose.cpp:105-125): [B,h,S,d] -> [B,S,h,d].
ORACLE_API void oracle_transpose_for_score(const float* in, float* out, int64_t B, int64_t S, int64_t h,
                                           int64_t d) {
#pragma omp parallel for
  for (int64_t idx = 0; idx < B * S; ++idx) {
    const int64_t b = idx / S, s = idx % S;
    for (int64_t head = 0; head < h; ++head)
      std::memcpy(out + ((b * S + s) * h + head) * d, in + ((b * h + head) * S + s) * d, d * sizeof(float));
  }
}

// kernels::TransposeForScorePad (layers/kernels/transpose.cpp:128-156): [B,h,maxS,d] ->
// packed [sum(len),h,d], pad rows skipped.
ORACLE_API void oracle_transpose_for_score_pad(const float* in, float* out, const int64_t* lens, int64_t B,
                                               int64_t maxS, int64_t h, int64_t d) {
#pragma omp parallel for
  for (int64_t idx = 0; idx < B * maxS; ++idx) {
    const int64_t b = idx / maxS, s = idx % maxS;
    if (s >= lens[b]) continue;
    const int64_t acc = std::accumulate(lens, lens + b, (int64_t)0);
    for (int64_t head = 0; head < h; ++head)
      std::memcpy(out + ((acc + s) * h + head) * d, in + ((b * h + head) * maxS + s) * d, d * sizeof(float));
  }
}

// kernels::ApplyMaskAndSoftmax -> SoftmaxMask (layers/kernels/softmax.cpp:28-81): five passes
// per row: x = qk*scale (+ mask), max, exp(x - max) with std::exp, sum, multiply by 1/sum.
// mask 2-D: mask[b, t]; 3-D: mask[b, f, t]; NULL: no add.
ORACLE_API void oracle_apply_mask_and_softmax(float* qk, const float* mask, int64_t B, int64_t h, int64_t F,
                                              int64_t T, float scale, int is_2d) {
  const int64_t M = B * h * F;
#pragma omp parallel for
  for (int64_t i = 0; i < M; ++i) {
    float* row = qk + i * T;
    if (mask) {
      const int64_t b = i / (h * F), f = i % F;
      const float* mrow = mask + (is_2d ? b * T : (b * F + f) * T);
      for (int64_t j = 0; j < T; ++j) row[j] = row[j] * scale + mrow[j];
    } else {
      for (int64_t j = 0; j < T; ++j) row[j] = row[j] * scale;
    }
    float mx = std::numeric_limits<float>::lowest();
    for (int64_t j = 0; j < T; ++j) mx = std::max(mx, row[j]);
    for (int64_t j = 0; j < T; ++j) row[j] = std::exp(row[j] - mx);
    float sum = 0;
    for (int64_t j = 0; j < T; ++j) sum += row[j];
    const float coef = 1.0f / sum;
    for (int64_t j = 0; j < T; ++j) row[j] *= coef;
  }
}

// kernels::LayerNorm (layers/kernels/layer_norm.cpp:43-74) and AddBiasLayerNorm (:130-164):
// single pass sum / sum of squares; var = E[x^2] - mean^2; out = beta + gamma * rstd * (x - mean).
ORACLE_API void oracle_add_bias_layer_norm(float* out, const float* input, const float* bias, const float* gamma,
                                           const float* beta, int64_t m, int64_t n, float eps) {
#pragma omp parallel for
  for (int64_t r = 0; r < m; ++r) {
    float mean = 0, var = 0;
    float* o = out + r * n;
    for (int64_t j = 0; j < n; ++j) {
      float t = o[j];
      if (input) t = o[j] = o[j] + input[r * n + j] + bias[j];
      mean += t;
      var += t * t;
    }
    mean = mean / n;
    var = var / n - mean * mean;
    var = 1.f / sqrtf(var + eps);
    for (int64_t j = 0; j < n; ++j) o[j] = beta[j] + gamma[j] * var * (o[j] - mean);
  }
}
ORACLE_API void oracle_layer_norm(float* out, const float* gamma, const float* beta, int64_t m, int64_t n,
                                  float eps) {
  oracle_add_bias_layer_norm(out, nullptr, nullptr, gamma, beta, m, n, eps);
}

// kernels::AddBiasAct<float, Gelu / Tanh / Relu> (layers/kernels/activation.cpp:33-88):
// gelu: x = out + bias; out = x * 0.5 * (1 + tanh(0.7978845608028654 * (x + 0.044715 x^3))).
ORACLE_API void oracle_add_bias_act(float* out, const float* bias, int64_t m, int64_t n, int act) {
#pragma omp parallel for
  for (int64_t r = 0; r < m; ++r) {
    float* o = out + r * n;
    for (int64_t j = 0; j < n; ++j) {
      const float x = o[j] + bias[j];
      if (act == 0) {
        const float u = 0.7978845608028654f * (x + 0.044715f * x * x * x);
        o[j] = x * 0.5f * (1.0f + std::tanh(u));
      } else if (act == 1) {
        o[j] = std::tanh(x);
      } else {
        o[j] = x > 0.f ? x : 0.f;
      }
    }
  }
}

// kernels::LookupEmbedding<Add> (layers/kernels/embedding.cpp:49-70). Returns -1 (and stops)
// on an id >= vocab, where the reference throws.
ORACLE_API int oracle_lookup_embedding(float* out, const float* table, const int64_t* ids, int64_t num_ids,
                                       int64_t hidden, int64_t vocab, int add) {
  for (int64_t i = 0; i < num_ids; ++i)
    if (ids[i] < 0 || ids[i] >= vocab) return -1;
#pragma omp parallel for
  for (int64_t i = 0; i < num_ids; ++i) {
    float* dst = out + i * hidden;
    const float* src = table + ids[i] * hidden;
    if (add) {
      for (int64_t j = 0; j < hidden; ++j) dst[j] += src[j];
    } else {
      std::copy(src, src + hidden, dst);
    }
  }
  return 0;
}

// layers::PrepareBertMasks (layers/prepare_bert_masks.cpp:24-66, kernels/common.cpp:76-81):
// default position ids 0..S-1 per row, token types 0, mask 1; ext = -10000 * (1 - mask).
ORACLE_API void oracle_prepare_bert_masks(int64_t B, int64_t S, int64_t* att_mask, int has_mask, int64_t* seq_type,
                                          int has_type, int64_t* pos_ids, int has_pos, float* ext_mask) {
  for (int64_t i = 0; i < B * S; ++i) {
    if (!has_pos) pos_ids[i] = i % S;
    if (!has_type) seq_type[i] = 0;
    if (!has_mask) att_mask[i] = 1;
    ext_mask[i] = -10000.0f * (1 - att_mask[i]);
  }
}

// ---------------------------------------------------------------------- layers ----------

// layers::BERTEmbedding::operator() (layers/bert_embedding.cpp:42-64):
// out = word[ids]; out += type[type_ids]; out += pos[pos_ids]; LayerNorm(out), eps 1e-12.
ORACLE_API int oracle_bert_embedding(float* out, const int64_t* ids, const int64_t* pos_ids,
                                     const int64_t* type_ids, const float* word, const float* pos,
                                     const float* type, const float* gamma, const float* beta, int64_t T,
                                     int64_t H, int64_t vocab, int64_t max_pos, int64_t num_types) {
  if (oracle_lookup_embedding(out, word, ids, T, H, vocab, 0) != 0) return -1;
  if (oracle_lookup_embedding(out, type, type_ids, T, H, num_types, 1) != 0) return -1;
  if (oracle_lookup_embedding(out, pos, pos_ids, T, H, max_pos, 1) != 0) return -1;
  oracle_layer_norm(out, gamma, beta, T, H, 1e-12f);
  return 0;
}

struct OracleLayerWeights {
  const float* qkv_w;   // [H,3H] = cat(Wq,Wk,Wv).T   (python layers/modeling_bert.py:184-191)
  const float* qkv_b;   // [3H]
  const float* attn_out_w;  // [H,H]  = W.T
  const float* attn_out_b;
  const float* attn_ln_g;
  const float* attn_ln_b;
  const float* inter_w;  // [H,F]
  const float* inter_b;
  const float* out_w;    // [F,H]
  const float* out_b;
  const float* out_ln_g;
  const float* out_ln_b;
};

// layers::BertAttention::operator() -> MultiHeadedAttention self path, post-LN
// (layers/bert_attention.cpp:29-47, layers/multi_headed_attention.cpp:168-205, 288-372).
// x[B,S,H], mask[B,1,1,S] or NULL -> out[B,S,H], attn[B,h,S,S].
ORACLE_API void oracle_bert_attention(const float* x, const float* mask, const OracleLayerWeights* w, int64_t B,
                                      int64_t S, int64_t H, int64_t heads, float* out, float* attn) {
  const int64_t T = B * S, d = H / heads;
  std::vector<float> qkv(T * 3 * H), q(T * H), k(T * H), v(T * H), ctx(T * H), merged(T * H);
  oracle_matmul(x, w->qkv_w, qkv.data(), T, 3 * H, H, 0, 1.f, 0.f);
  oracle_split_add_bias_transpose(qkv.data(), w->qkv_b, q.data(), k.data(), v.data(), B, S, heads, d);
  const float scaler = 1.0f / std::sqrt((float)d);
  oracle_batch_matmul(q.data(), k.data(), attn, B * heads, S, S, d, 1, scaler, 0.f);
  oracle_apply_mask_and_softmax(attn, mask, B, heads, S, S, 1.0f, 1);
  oracle_batch_matmul(attn, v.data(), ctx.data(), B * heads, S, d, S, 0, 1.f, 0.f);
  oracle_transpose_for_score(ctx.data(), merged.data(), B, S, heads, d);
  oracle_matmul(merged.data(), w->attn_out_w, out, T, H, H, 0, 1.f, 0.f);
  oracle_add_bias_layer_norm(out, x, w->attn_out_b, w->attn_ln_g, w->attn_ln_b, T, H, 1e-12f);
}

// layers::MultiHeadedAttentionSmartBatch self path (layers/multi_headed_attention_smart_batch.cpp
// :186-219, 304-412): x packed [sum(len),H]; mask[B,1,maxS] (-1e9 on pad keys) or NULL;
// out packed [sum(len),H]; attn padded [B,h,maxS,maxS].
ORACLE_API void oracle_smart_attention(const float* x, const float* mask, const OracleLayerWeights* w,
                                       const int64_t* lens, int64_t B, int64_t H, int64_t heads, float* out,
                                       float* attn) {
  const int64_t total = std::accumulate(lens, lens + B, (int64_t)0);
  const int64_t maxS = *std::max_element(lens, lens + B), d = H / heads;
  std::vector<float> qkv(total * 3 * H), q(B * maxS * H), k(B * maxS * H), v(B * maxS * H), ctx(B * maxS * H),
      merged(total * H);
  oracle_matmul(x, w->qkv_w, qkv.data(), total, 3 * H, H, 0, 1.f, 0.f);
  oracle_split_add_bias_transpose_pad(qkv.data(), w->qkv_b, q.data(), k.data(), v.data(), lens, B, maxS, heads, d);
  const float scaler = 1.0f / std::sqrt((float)d);
  oracle_batch_matmul(q.data(), k.data(), attn, B * heads, maxS, maxS, d, 1, scaler, 0.f);
  oracle_apply_mask_and_softmax(attn, mask, B, heads, maxS, maxS, 1.0f, 1);
  oracle_batch_matmul(attn, v.data(), ctx.data(), B * heads, maxS, d, maxS, 0, 1.f, 0.f);
  oracle_transpose_for_score_pad(ctx.data(), merged.data(), lens, B, maxS, heads, d);
  oracle_matmul(merged.data(), w->attn_out_w, out, total, H, H, 0, 1.f, 0.f);
  oracle_add_bias_layer_norm(out, x, w->attn_out_b, w->attn_ln_g, w->attn_ln_b, total, H, 1e-12f);
}

// layers::BertIntermediate (layers/bert_intermediate.cpp:38-46) + layers::BertOutput
// (layers/bert_output.cpp:41-51); the same pair is layers::AlbertLayer (albert_layer.cpp:34-49).
ORACLE_API void oracle_bert_ffn(const float* a, const OracleLayerWeights* w, int64_t T, int64_t H, int64_t F,
                                float* inter, float* out) {
  oracle_matmul(a, w->inter_w, inter, T, F, H, 0, 1.f, 0.f);
  oracle_add_bias_act(inter, w->inter_b, T, F, 0);
  oracle_matmul(inter, w->out_w, out, T, H, F, 0, 1.f, 0.f);
  oracle_add_bias_layer_norm(out, a, w->out_b, w->out_ln_g, w->out_ln_b, T, H, 1e-12f);
}

// One encoder layer = BertAttention -> BertIntermediate -> BertOutput
// (python layers/modeling_bert.py:238-259; example/cpp/bert_model.cpp:68-79).
ORACLE_API void oracle_bert_layer(const float* x, const float* mask, const OracleLayerWeights* w, int64_t B,
                                  int64_t S, int64_t H, int64_t heads, int64_t F, float* out, float* attn) {
  const int64_t T = B * S;
  std::vector<float> a(T * H), inter(T * F);
  oracle_bert_attention(x, mask, w, B, S, H, heads, a.data(), attn);
  oracle_bert_ffn(a.data(), w, T, H, F, inter.data(), out);
}

ORACLE_API void oracle_smart_layer(const float* x, const float* mask, const OracleLayerWeights* w,
                                   const int64_t* lens, int64_t B, int64_t H, int64_t heads, int64_t F,
                                   float* out, float* attn) {
  const int64_t total = std::accumulate(lens, lens + B, (int64_t)0);
  std::vector<float> a(total * H), inter(total * F);
  oracle_smart_attention(x, mask, w, lens, B, H, heads, a.data(), attn);
  oracle_bert_ffn(a.data(), w, total, H, F, inter.data(), out);
}

// Encoder stack on an embedded input: hidden = layer_L(...layer_1(x)) (modeling_bert.py:284-322).
// `attn_scratch` holds one layer's [B,h,S,S] probabilities.
ORACLE_API void oracle_bert_encoder(const float* x, const float* mask, const OracleLayerWeights* layers,
                                    int64_t num_layers, int64_t B, int64_t S, int64_t H, int64_t heads, int64_t F,
                                    float* out, float* attn_scratch) {
  const int64_t T = B * S;
  std::vector<float> cur(x, x + T * H), nxt(T * H);
  for (int64_t l = 0; l < num_layers; ++l) {
    oracle_bert_layer(cur.data(), mask, &layers[l], B, S, H, heads, F, nxt.data(), attn_scratch);
    cur.swap(nxt);
  }
  std::copy(cur.begin(), cur.end(), out);
}

// --------------------------------------------------------------- int8 Linear (config 5) --
// Not a restatement of reference code: the reference delegates int8 to torch dynamic
// quantisation.  This is the scheme the benchmark configuration states:
//   s_x = max|x| / 127 (per tensor), q_x = clamp(rint(x / s_x), -127, 127)
//   s_w[n] = max_k |w[n,k]| / 127 (per output channel), q_w likewise
//   acc[m,n] = sum_k q_x[m,k] * q_w[n,k]  (int32, exact);  y = acc * s_x * s_w[n] + b[n]
ORACLE_API float oracle_quantize_tensor_i8(const float* x, int8_t* q, int64_t n) {
  float mx = 0.f;
  for (int64_t i = 0; i < n; ++i) mx = std::max(mx, std::fabs(x[i]));
  const float scale = mx > 0.f ? mx / 127.0f : 1.0f;
  for (int64_t i = 0; i < n; ++i) {
    float r = std::nearbyintf(x[i] / scale);
    r = std::min(std::max(r, -127.f), 127.f);
    q[i] = (int8_t)r;
  }
  return scale;
}
ORACLE_API void oracle_quantize_weight_i8(const float* w, int8_t* q, float* scales, int64_t N, int64_t K) {
  for (int64_t n = 0; n < N; ++n) scales[n] = oracle_quantize_tensor_i8(w + n * K, q + n * K, K);
}
ORACLE_API void oracle_gemm_i8(const int8_t* A, const int8_t* B, int32_t* C, int64_t M, int64_t N, int64_t K) {
#pragma omp parallel for
  for (int64_t m = 0; m < M; ++m)
    for (int64_t n = 0; n < N; ++n) {
      int32_t acc = 0;
      for (int64_t k = 0; k < K; ++k) acc += (int32_t)A[m * K + k] * (int32_t)B[n * K + k];
      C[m * N + n] = acc;
    }
}
ORACLE_API void oracle_dequant_bias(const int32_t* acc, float act_scale, const float* w_scale, const float* bias,
                                    float* out, int64_t M, int64_t N) {
  for (int64_t i = 0; i < M * N; ++i) {
    float v = (float)acc[i] * act_scale * w_scale[i % N];
    if (bias) v += bias[i % N];
    out[i] = v;
  }
}
