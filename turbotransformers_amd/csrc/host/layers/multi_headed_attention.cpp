#include "layers/multi_headed_attention.h"

#include <cmath>

#include "core/device_context.h"
#include "layers/kernels.h"
#include "ttmi.h"

namespace turbo_transformers {
namespace layers {

using core::DeviceContext;
using core::Tensor;

static void* Stream() { return DeviceContext::GetInstance().stream(); }

void MultiHeadedAttention::EnforceShapeAndType() const {
  TT_ENFORCE(!qkv_weight_.is_null() && !qkv_bias_.is_null(), "self attention needs the fused qkv weight and bias");
  TT_ENFORCE_EQ(qkv_weight_.n_dim(), (size_t)2, "qkv_weight must be a matrix");
  TT_ENFORCE_EQ(dense_weight_.n_dim(), (size_t)2, "dense_weight must be a matrix");
  TT_ENFORCE_EQ(dense_weight_.shape(0), dense_weight_.shape(1), "dense_weight must be [hidden, hidden]");
  const int64_t hidden = dense_weight_.shape(0);
  TT_ENFORCE_EQ(qkv_weight_.numel(), 3 * hidden * hidden, "qkv_weight must hold 3*hidden*hidden elements");
  TT_ENFORCE_EQ(qkv_bias_.numel(), 3 * hidden, "qkv_bias must hold 3*hidden elements");
  TT_ENFORCE_EQ(dense_bias_.numel(), hidden, "dense_bias must hold hidden elements");
  TT_ENFORCE(num_attention_heads_ > 0 && hidden % num_attention_heads_ == 0, "hidden must be a multiple of the head count");
  TT_ENFORCE(core::SameDataType(qkv_weight_.dtype(), dense_weight_.dtype()), "weights must share one element type");
}

void BertAttention::EnforceShapeAndType() const {
  MultiHeadedAttention::EnforceShapeAndType();
  TT_ENFORCE(!layernorm_gamma_.is_null() && !layernorm_beta_.is_null(), "BertAttention needs LayerNorm parameters");
  TT_ENFORCE_EQ(layernorm_gamma_.numel(), dense_weight_.shape(0), "LayerNorm weight size mismatch");
  TT_ENFORCE_EQ(layernorm_beta_.numel(), dense_weight_.shape(0), "LayerNorm bias size mismatch");
}

bool MultiHeadedAttention::UseFusedCore(const Tensor& attention_mask, const Tensor* att_score, int64_t head_dim, int dtype,
                                        int64_t batch, int64_t seq, int64_t heads) {
  bool mask_is_key_mask = true;
  if (!attention_mask.is_null()) {
    mask_is_key_mask = attention_mask.n_dim() == 2 || (attention_mask.n_dim() == 3 && attention_mask.shape(1) == 1) ||
                       (attention_mask.n_dim() == 4 && attention_mask.shape(2) == 1);
  }
  bool dtype_ok = dtype == TTMI_F16 || dtype == TTMI_BF16;
  if (dtype == TTMI_F32 && batch > 0) {
    // the fp32 kernel is bound by the matrix pipe: a wavefront's 32 queries cost 3.4 us per 64 keys.  It beats the
    // three launches of the chain (18 us) when the sequence is short or when there are wavefronts for half the SIMDs
    // (1024 on this chip).  (batch, seq: of the padded tensors when the batch is a packed one)
    const int64_t wave_blocks = batch * heads * ((seq + 31) / 32);
    dtype_ok = seq <= 128 || wave_blocks >= 512;
  }
  return att_score == nullptr && head_dim == 64 && dtype_ok && mask_is_key_mask;
}

static int64_t RoundUp8(int64_t n) { return (n + 7) / 8 * 8; }

// score -> softmax -> P V -> merge heads -> output projection -> bias (+input) (+LayerNorm)
void MultiHeadedAttention::AttentionTail(const Tensor& query_tensor, const Tensor& attention_mask, Tensor* output,
                                         Tensor* att_score, int64_t batch, int64_t seq, int64_t key_seq, const Tensor& k,
                                         const Tensor& v, const std::vector<int64_t>* seq_list, bool fused_core, int64_t v_pitch,
                                         bool post_layernorm, bool post_add_input, bool is_trans_weight) const {
  const int dt = kernels::DeviceDType(query_tensor);
  const DLDeviceType dev = query_tensor.device_type();
  const int dev_id = query_tensor.device_id();
  const int64_t hidden = query_tensor.shape(-1), heads = num_attention_heads_, d = hidden / heads;
  const int64_t tokens = query_tensor.numel() / hidden;

  ctx_.ReshapeAs(query_tensor.dtype(), {tokens, hidden}, dev, dev_id, "batch_gemm4/Reshape");
  const float scaler = 1.0f / std::sqrt(static_cast<float>(d));

  // Nobody asked for the probabilities: run the whole core as one kernel; the [B,h,S,S] scores
  // never reach HBM.
  if (fused_core) {
    const float* mask = nullptr;
    if (!attention_mask.is_null()) {
      TT_ENFORCE_EQ(attention_mask.numel(), batch * seq, "attention mask has the wrong size");
      mask = attention_mask.data<float>();
    }
    TT_ENFORCE_EQ(seq, key_seq, "the fused core is for self attention without a key/value cache");
    const int32_t* cu = nullptr;
    if (seq_list != nullptr) cu = DeviceContext::GetInstance().GetSeqPlan(*seq_list).cu_seqlens;
    TT_DEVICE_CALL(ttmi_fused_attention(q_.raw(), k.raw(), v.raw(), mask, ctx_.mutable_raw(), cu, batch, heads, seq, d,
                                        v_pitch, scaler, dt, Stream()));
  } else {
  Tensor* score = att_score != nullptr ? att_score : &score_scratch_;
  // score is [B,h,F,T]: F = query positions, T = key positions (they differ for context attention
  // and when a key/value cache has been prepended)
  const int64_t F = seq, T = key_seq;
  score->ReshapeAs(query_tensor.dtype(), {batch, heads, F, T}, dev, dev_id, "batch_gemm3/Reshape");
  // batch_gemm3: score[b,h] = scaler * q[b,h] k[b,h]^T   (multi_headed_attention.cpp:328-330)
  TT_DEVICE_CALL(ttmi_gemm_strided_batched(q_.raw(), k.raw(), score->mutable_raw(), F, T, d, d, d, T, F * d, T * d, F * T,
                                           batch * heads, 1, scaler, 0.f, dt, Stream()));
  kernels::ApplyMaskAndSoftmax(score, attention_mask, 1.0f);

  if (seq_list == nullptr) {
    // batch_gemm4 with the [B,h,F,d] -> [B,F,h,d] transpose folded into the store (:345-354)
    TT_DEVICE_CALL(ttmi_gemm_batched_heads(score->raw(), v.raw(), ctx_.mutable_raw(), F, d, T, T, d, hidden, heads,
                                           heads * F * T, F * T, heads * T * d, T * d, F * hidden, d, batch, 0, 1.f, 0.f, dt,
                                           Stream()));
  } else {
    // padded P V, then drop the pad rows while merging heads (…smart_batch.cpp:385-392)
    Tensor& padded = ln_query_;  // free at this point of the call
    padded.ReshapeAs(query_tensor.dtype(), {batch, heads, seq, d}, dev, dev_id, "ApplyMaskAndSoftmax/Reshape");
    TT_DEVICE_CALL(ttmi_gemm_strided_batched(score->raw(), v.raw(), padded.mutable_raw(), seq, d, seq, seq, d, d, seq * seq,
                                             seq * d, seq * d, batch * heads, 0, 1.f, 0.f, dt, Stream()));
    kernels::TransposeForScorePad(&ctx_, padded, *seq_list);
  }
  }  // unfused core

  output->ReshapeAs(query_tensor.dtype(), {query_tensor.shape(0), query_tensor.shape(1), hidden}, dev, dev_id, "gemm5/Reshape");
  const void* wo = dense_packed_.Get(dense_weight_, is_trans_weight);
  if (!post_add_input && post_layernorm) {
    // gemm5 then AddBiasLayerNorm(query, bias, gamma, beta, out), eps 1e-12 (:359-371)
    kernels::GemmAddBiasLayerNorm(ctx_, wo, hidden, query_tensor, dense_bias_, layernorm_gamma_, layernorm_beta_, output, 1e-12f);
  } else {
    ttmi_epilogue_args args{};
    args.bias = dense_bias_.raw();
    args.residual = post_add_input ? query_tensor.raw() : nullptr;
    TT_DEVICE_CALL(ttmi_gemm_fused(ctx_.raw(), wo, output->mutable_raw(), tokens, hidden, hidden, hidden, hidden, hidden,
                                   post_add_input ? TTMI_EPI_BIAS_RESIDUAL : TTMI_EPI_BIAS, &args, dt, Stream()));
  }
}

// One projection followed by AddBiasTransposeForScore, as one GEMM: x[B,S,H] W + b -> [B,h,S,d]
// (multi_headed_attention.cpp:73-88, :107-150).
static void ProjectToHeads(const Tensor& x, const void* packed_w, const Tensor& bias, int64_t heads, Tensor* out,
                           const char* name) {
  const int64_t batch = x.shape(0), seq = x.shape(1), hidden = x.shape(2), d = hidden / heads;
  out->ReshapeAs(x.dtype(), {batch, heads, seq, d}, x.device_type(), x.device_id(), name);
  ttmi_epilogue_args args{};
  args.bias = bias.raw();
  args.q = out->mutable_raw();
  args.seq = seq;
  args.heads = heads;
  args.head_dim = d;
  TT_DEVICE_CALL(ttmi_gemm_fused(x.raw(), packed_w, nullptr, batch * seq, hidden, hidden, hidden, hidden, hidden,
                                 TTMI_EPI_QKV_SPLIT, &args, kernels::DeviceDType(x), Stream()));
}

static bool CacheHas(const std::unordered_map<std::string, Tensor*>& cache, const char* key) {
  auto it = cache.find(key);
  return it != cache.end() && it->second != nullptr && !it->second->is_null();
}

// cache[key] = a copy of `src` (multi_headed_attention.cpp:216-229)
static void StoreInCache(std::unordered_map<std::string, Tensor*>& cache, const char* key, const Tensor& src, const char* name) {
  auto it = cache.find(key);
  TT_ENFORCE(it != cache.end() && it->second != nullptr, "layer_cache has no entry %s", key);
  std::vector<int64_t> shape;
  for (size_t i = 0; i < src.n_dim(); ++i) shape.push_back(src.shape((int)i));
  it->second->ReshapeAs(src.dtype(), shape, src.device_type(), src.device_id(), name);
  core::CopyBytes(it->second->mutable_raw(), src.device_type(), src.raw(), src.device_type(),
                  (size_t)src.numel() * src.element_size());
}

void MultiHeadedAttention::operator()(const Tensor& key_tensor, const Tensor& value_tensor, const Tensor& query_tensor,
                                      const Tensor& attention_mask, const std::string& attn_type, Tensor* output,
                                      Tensor* att_score, std::unordered_map<std::string, Tensor*> layer_cache,
                                      bool pre_layernorm, bool post_layernorm, bool post_add_input,
                                      bool is_trans_weight) const {
  std::lock_guard<std::mutex> g(mutex_);
  const bool is_self = attn_type == "self";
  TT_ENFORCE(is_self || attn_type == "context", "attn_type should be context or self.");
  TT_ENFORCE_EQ(query_tensor.n_dim(), (size_t)3, "The query_tensors should be a matrix with shape [batch_size, query_seq_len, hidden_size].");
  TT_ENFORCE(output != nullptr, "output must not be null");
  kernels::RequireGpu(query_tensor, "MultiHeadedAttention");
  TT_ENFORCE_EQ(dense_weight_.n_dim(), (size_t)2, "dense_weight must be a matrix");

  const int64_t batch = query_tensor.shape(0), seq = query_tensor.shape(1), hidden = query_tensor.shape(2);
  TT_ENFORCE_EQ(hidden, dense_weight_.shape(0), "hidden size of the input and of the weights differ");
  TT_ENFORCE(core::SameDataType(query_tensor.dtype(), dense_weight_.dtype()), "input and weights must share one element type");
  const int64_t heads = num_attention_heads_, d = hidden / heads;
  TT_ENFORCE(heads > 0 && hidden % heads == 0, "hidden must be a multiple of the head count");
  const int dt = kernels::DeviceDType(query_tensor);
  const DLDeviceType dev = query_tensor.device_type();
  const int dev_id = query_tensor.device_id();
  for (const auto& kv : layer_cache) {
    if (kv.second == nullptr || kv.second->is_null()) continue;
    kernels::RequireGpu(*kv.second, "layer_cache");
    TT_ENFORCE(core::SameDataType(kv.second->dtype(), query_tensor.dtype()), "layer_cache[%s] and the query differ in element type", kv.first.c_str());
    TT_ENFORCE(kv.second->n_dim() == 4 && kv.second->shape(0) == batch && kv.second->shape(1) == heads && kv.second->shape(3) == d,
               "layer_cache[%s] must be [batch, heads, len, head_dim]", kv.first.c_str());
  }

  const Tensor* q_in = &query_tensor;
  if (pre_layernorm) {  // :66-80, :190-199 -- eps is 1e-6 there
    TT_ENFORCE(!layernorm_gamma_.is_null() && !layernorm_beta_.is_null(), "pre_layernorm needs LayerNorm parameters");
    ln_query_.ReshapeAs(query_tensor.dtype(), {batch, seq, hidden}, dev, dev_id, "self/layernorm/Reshape");
    core::CopyBytes(ln_query_.mutable_raw(), dev, query_tensor.raw(), dev, (size_t)query_tensor.numel() * query_tensor.element_size());
    kernels::LayerNorm<float>(layernorm_gamma_, layernorm_beta_, &ln_query_, 1e-6f);
    q_in = &ln_query_;
  }

  const Tensor* k_used = &k_;
  const Tensor* v_used = &v_;
  int64_t v_pitch = 0;
  bool fused_core = false;
  if (is_self) {
    MultiHeadedAttention::EnforceShapeAndType();
    // with the fused core V is kept transposed, [B,h,d,pitch]: its tiles are then plain copies.
    // A key/value cache needs the row-major layout (it is appended along the sequence).
    // (fp32 with up to 192 rows keeps V row-major: that QKV projection is cut along K, which the transposed-V
    // epilogue cannot be, and the fp32 kernel takes either layout)
    const bool fused_self = layer_cache.empty() && UseFusedCore(attention_mask, att_score, d, dt, batch, seq, heads);
    if (fused_self && !(dt == TTMI_F32 && batch * seq <= 192)) v_pitch = RoundUp8(seq);
    fused_core = fused_self;
    q_.ReshapeAs(query_tensor.dtype(), {batch, heads, seq, d}, dev, dev_id, "self/q/Reshape");
    k_.ReshapeAs(query_tensor.dtype(), {batch, heads, seq, d}, dev, dev_id, "self/k/Reshape");
    if (v_pitch > 0) v_.ReshapeAs(query_tensor.dtype(), {batch, heads, d, v_pitch}, dev, dev_id, "self/v/Reshape");
    else v_.ReshapeAs(query_tensor.dtype(), {batch, heads, seq, d}, dev, dev_id, "self/v/Reshape");
    // gemm012_fused + SplitAddBiasTransposeForScore in one launch (:199-203)
    ttmi_epilogue_args args{};
    args.bias = qkv_bias_.raw();
    args.q = q_.mutable_raw();
    args.k = k_.mutable_raw();
    args.v = v_.mutable_raw();
    args.seq = seq;
    args.heads = heads;
    args.head_dim = d;
    args.v_seq_pitch = v_pitch;
    TT_DEVICE_CALL(ttmi_gemm_fused(q_in->raw(), qkv_packed_.Get(qkv_weight_, is_trans_weight), nullptr, batch * seq, 3 * hidden,
                                   hidden, hidden, hidden, 3 * hidden, TTMI_EPI_QKV_SPLIT, &args, dt, Stream()));
    // decoder self attention: earlier keys/values come first (:205-214), the grown tensors go back (:216-229)
    auto prepend = [&](const char* key, Tensor* cur, Tensor* grown, const char* name) {
      if (!CacheHas(layer_cache, key)) return;
      const Tensor& past = *layer_cache.at(key);
      const int64_t past_len = past.shape(2);
      grown->ReshapeAs(query_tensor.dtype(), {batch, heads, past_len + seq, d}, dev, dev_id, name);
      TT_DEVICE_CALL(ttmi_concat(past.raw(), cur->raw(), grown->mutable_raw(), batch * heads, past_len * d, seq * d, dt, Stream()));
      std::swap(*cur, *grown);
    };
    prepend("self_keys", &k_, &k_grown_, "self/keys/Concat");
    prepend("self_values", &v_, &v_grown_, "self/values/Concat");
    if (!layer_cache.empty()) {
      StoreInCache(layer_cache, "self_keys", k_, "self/self_key/Reshape");
      StoreInCache(layer_cache, "self_values", v_, "self/self_value/Reshape");
    }
  } else {
    TT_ENFORCE(!q_weight_.is_null() && !k_weight_.is_null() && !v_weight_.is_null() && !q_bias_.is_null() && !k_bias_.is_null() &&
                   !v_bias_.is_null(), "context attention needs the separate q/k/v weights and biases");
    ProjectToHeads(*q_in, q_packed_.Get(q_weight_, is_trans_weight), q_bias_, heads, &q_, "context/AddBiasTransposeForScore/q_out2/Reshape");
    if (CacheHas(layer_cache, "memory_keys") && CacheHas(layer_cache, "memory_values")) {
      // the encoder memory was projected at an earlier step (:90-105); used in place, no copy
      k_used = layer_cache.at("memory_keys");
      v_used = layer_cache.at("memory_values");
    } else {
      TT_ENFORCE_EQ(key_tensor.n_dim(), (size_t)3, "The key_tensor should be a matrix with shape [batch_size, key_seq_len, hidden_size].");
      TT_ENFORCE_EQ(value_tensor.n_dim(), (size_t)3, "The value_tensor should be a matrix with shape [batch_size, key_seq_len, hidden_size].");
      kernels::RequireGpu(key_tensor, "MultiHeadedAttention");
      kernels::RequireGpu(value_tensor, "MultiHeadedAttention");
      TT_ENFORCE(key_tensor.shape(0) == batch && value_tensor.shape(0) == batch && key_tensor.shape(1) == value_tensor.shape(1) &&
                     key_tensor.shape(2) == hidden && value_tensor.shape(2) == hidden,
                 "key and value must be [batch_size, key_seq_len, hidden_size]");
      TT_ENFORCE(core::SameDataType(key_tensor.dtype(), query_tensor.dtype()) && core::SameDataType(value_tensor.dtype(), query_tensor.dtype()),
                 "key, value and query must share one element type");
      ProjectToHeads(key_tensor, k_packed_.Get(k_weight_, is_trans_weight), k_bias_, heads, &k_, "context/keys/AddBiasTransposeForScore/Reshape");
      ProjectToHeads(value_tensor, v_packed_.Get(v_weight_, is_trans_weight), v_bias_, heads, &v_, "context/values/AddBiasTransposeForScore/Reshape");
      if (!layer_cache.empty()) {  // :128-150
        StoreInCache(layer_cache, "memory_keys", k_, "context/keys/AddBiasTransposeForScore/Reshape");
        StoreInCache(layer_cache, "memory_values", v_, "context/values/AddBiasTransposeForScore/Reshape");
      }
    }
  }
  const int64_t key_seq = fused_core ? seq : k_used->shape(2);
  TT_ENFORCE_EQ(fused_core ? seq : v_used->shape(2), key_seq, "keys and values differ in length");

  AttentionTail(query_tensor, attention_mask, output, att_score, batch, seq, key_seq, *k_used, *v_used, nullptr, fused_core, v_pitch,
                post_layernorm, post_add_input, is_trans_weight);
}

void BertAttention::operator()(const Tensor& input_tensor, const Tensor& attention_mask, Tensor* output, Tensor* attn,
                               bool is_trans_weight) const {
  // bert_attention.cpp:29-47: self attention, post-LayerNorm, no extra residual
  std::unordered_map<std::string, Tensor*> dummy{};
  MultiHeadedAttention::operator()(input_tensor, input_tensor, input_tensor, attention_mask, "self", output, attn, dummy,
                                   false /* pre_layernorm */, true /* post_layernorm */, false /* post_add_input */,
                                   is_trans_weight);
}

void MultiHeadedAttentionSmartBatch::operator()(const Tensor& key_tensor, const Tensor& value_tensor,
                                                const Tensor& query_tensor, const Tensor& attention_mask,
                                                const std::string& attn_type, Tensor* output, Tensor* att_score,
                                                std::unordered_map<std::string, Tensor*> layer_cache,
                                                const std::vector<int64_t>& query_seq_len_list,
                                                const std::vector<int64_t>& key_seq_len_list, bool pre_layernorm,
                                                bool post_layernorm, bool post_add_input, bool is_trans_weight) const {
  std::lock_guard<std::mutex> g(mutex_);
  TT_ENFORCE(attn_type == "self", "only attn_type \"self\" is built (\"context\" belongs to the decoder path)");
  TT_ENFORCE(layer_cache.empty(), "layer_cache belongs to the decoder path and is not built");
  TT_ENFORCE(!pre_layernorm, "pre_layernorm is not built for the smart-batch layer");
  TT_ENFORCE_EQ(query_tensor.n_dim(), (size_t)3, "The query_tensors should be a matrix with shape [1, sum_query_seq_len, hidden_size].");
  TT_ENFORCE_EQ(query_tensor.shape(0), (int64_t)1, "a packed batch has leading dimension 1");
  TT_ENFORCE(output != nullptr, "output must not be null");
  kernels::RequireGpu(query_tensor, "MultiHeadedAttentionSmartBatch");
  MultiHeadedAttention::EnforceShapeAndType();
  (void)key_tensor;
  (void)value_tensor;
  (void)key_seq_len_list;

  auto plan = DeviceContext::GetInstance().GetSeqPlan(query_seq_len_list);
  TT_ENFORCE_EQ(query_tensor.shape(1), plan.total, "The query_tensor shape 1 should be the sum of seq_len_list.");
  const int64_t hidden = query_tensor.shape(2), heads = num_attention_heads_, d = hidden / heads;
  TT_ENFORCE_EQ(hidden, dense_weight_.shape(0), "hidden size of the input and of the weights differ");
  TT_ENFORCE(core::SameDataType(query_tensor.dtype(), qkv_weight_.dtype()), "input and weights must share one element type");
  const int dt = kernels::DeviceDType(query_tensor);
  const DLDeviceType dev = query_tensor.device_type();
  const int dev_id = query_tensor.device_id();
  const int64_t batch = plan.batch, max_seq = plan.max_seq;

  // Padded q,k,v; the QKV GEMM scatters bias-added rows of the packed input into them.  The
  // unfused core multiplies whole padded tensors, so pad rows must be exactly 0 there
  // (transpose.cpp:504-522); the fused kernel never reads a pad row, so nothing is cleared.
  // V stays row-major here: the transposed store needs the row map and a division per group of eight packed rows,
  // and that costs the QKV GEMM more than the scatter costs the attention kernel (20 requests, 6275 tokens:
  // 2.50 against 2.39 ms per forward).
  const bool fused_core = UseFusedCore(attention_mask, att_score, d, dt, batch, max_seq, heads);
  Tensor* qkv[3] = {&q_, &k_, &v_};
  const char* names[3] = {"self/q/Reshape", "self/k/Reshape", "self/v/Reshape"};
  for (int i = 0; i < 3; ++i) {
    qkv[i]->ReshapeAs(query_tensor.dtype(), {batch, heads, max_seq, d}, dev, dev_id, names[i]);
    if (fused_core) continue;
    const size_t bytes = (size_t)qkv[i]->numel() * qkv[i]->element_size();
    TT_DEVICE_CALL(ttmi_memset_zero(qkv[i]->mutable_raw(), (bytes + 3) / 4 * 4  /* capacity is rounded to 512 B */, Stream()));
  }
  ttmi_epilogue_args args{};
  args.bias = qkv_bias_.raw();
  args.q = q_.mutable_raw();
  args.k = k_.mutable_raw();
  args.v = v_.mutable_raw();
  args.seq = max_seq;
  args.heads = heads;
  args.head_dim = d;
  args.token_rows = plan.token_rows;
  args.batch = batch;
  TT_DEVICE_CALL(ttmi_gemm_fused(query_tensor.raw(), qkv_packed_.Get(qkv_weight_, is_trans_weight), nullptr, plan.total,
                                 3 * hidden, hidden, hidden, hidden, 3 * hidden, TTMI_EPI_QKV_SPLIT_PAD, &args, dt, Stream()));

  AttentionTail(query_tensor, attention_mask, output, att_score, batch, max_seq, max_seq, k_, v_, &query_seq_len_list, fused_core, 0,
                post_layernorm, post_add_input, is_trans_weight);
}

}  // namespace layers
}  // namespace turbo_transformers
