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

bool MultiHeadedAttention::UseFusedCore(const Tensor& attention_mask, const Tensor* att_score, int64_t head_dim, int dtype) {
  bool mask_is_key_mask = true;
  if (!attention_mask.is_null()) {
    mask_is_key_mask = attention_mask.n_dim() == 2 || (attention_mask.n_dim() == 3 && attention_mask.shape(1) == 1) ||
                       (attention_mask.n_dim() == 4 && attention_mask.shape(2) == 1);
  }
  return att_score == nullptr && head_dim == 64 && (dtype == TTMI_F16 || dtype == TTMI_BF16) && mask_is_key_mask;
}

static int64_t RoundUp8(int64_t n) { return (n + 7) / 8 * 8; }

// score -> softmax -> P V -> merge heads -> output projection -> bias (+input) (+LayerNorm)
void MultiHeadedAttention::SelfAttentionTail(const Tensor& query_tensor, const Tensor& attention_mask, Tensor* output,
                                             Tensor* att_score, int64_t batch, int64_t seq,
                                             const std::vector<int64_t>* seq_list, int64_t v_pitch, bool post_layernorm,
                                             bool post_add_input, bool is_trans_weight) const {
  const int dt = kernels::DeviceDType(query_tensor);
  const DLDeviceType dev = query_tensor.device_type();
  const int dev_id = query_tensor.device_id();
  const int64_t hidden = query_tensor.shape(-1), heads = num_attention_heads_, d = hidden / heads;
  const int64_t tokens = query_tensor.numel() / hidden;

  ctx_.ReshapeAs(query_tensor.dtype(), {tokens, hidden}, dev, dev_id, "batch_gemm4/Reshape");
  const float scaler = 1.0f / std::sqrt(static_cast<float>(d));

  // Nobody asked for the probabilities: run the whole core as one kernel; the [B,h,S,S] scores
  // never reach HBM.
  if (v_pitch > 0) {
    const float* mask = nullptr;
    if (!attention_mask.is_null()) {
      TT_ENFORCE_EQ(attention_mask.numel(), batch * seq, "attention mask has the wrong size");
      mask = attention_mask.data<float>();
    }
    const int32_t* cu = nullptr;
    if (seq_list != nullptr) cu = DeviceContext::GetInstance().GetSeqPlan(*seq_list).cu_seqlens;
    TT_DEVICE_CALL(ttmi_fused_attention(q_.raw(), k_.raw(), v_.raw(), mask, ctx_.mutable_raw(), cu, batch, heads, seq, d,
                                        v_pitch, scaler, dt, Stream()));
  } else {
  Tensor* score = att_score != nullptr ? att_score : &score_scratch_;
  score->ReshapeAs(query_tensor.dtype(), {batch, heads, seq, seq}, dev, dev_id, "batch_gemm3/Reshape");
  // batch_gemm3: score[b,h] = scaler * q[b,h] k[b,h]^T   (multi_headed_attention.cpp:328-330)
  TT_DEVICE_CALL(ttmi_gemm_strided_batched(q_.raw(), k_.raw(), score->mutable_raw(), seq, seq, d, d, d, seq, seq * d,
                                           seq * d, seq * seq, batch * heads, 1, scaler, 0.f, dt, Stream()));
  kernels::ApplyMaskAndSoftmax(score, attention_mask, 1.0f);

  if (seq_list == nullptr) {
    // batch_gemm4 with the [B,h,S,d] -> [B,S,h,d] transpose folded into the store (:345-354)
    TT_DEVICE_CALL(ttmi_gemm_batched_heads(score->raw(), v_.raw(), ctx_.mutable_raw(), seq, d, seq, seq, d, hidden, heads,
                                           heads * seq * seq, seq * seq, heads * seq * d, seq * d, seq * hidden, d, batch, 0,
                                           1.f, 0.f, dt, Stream()));
  } else {
    // padded P V, then drop the pad rows while merging heads (…smart_batch.cpp:385-392)
    Tensor& padded = ln_query_;  // free at this point of the call
    padded.ReshapeAs(query_tensor.dtype(), {batch, heads, seq, d}, dev, dev_id, "ApplyMaskAndSoftmax/Reshape");
    TT_DEVICE_CALL(ttmi_gemm_strided_batched(score->raw(), v_.raw(), padded.mutable_raw(), seq, d, seq, seq, d, d, seq * seq,
                                             seq * d, seq * d, batch * heads, 0, 1.f, 0.f, dt, Stream()));
    kernels::TransposeForScorePad(&ctx_, padded, *seq_list);
  }
  }  // unfused core

  output->ReshapeAs(query_tensor.dtype(), {query_tensor.shape(0), query_tensor.shape(1), hidden}, dev, dev_id, "gemm5/Reshape");
  const void* wo = dense_packed_.Get(dense_weight_, is_trans_weight);
  if (!post_add_input && post_layernorm) {
    // gemm5 then AddBiasLayerNorm(query, bias, gamma, beta, out), eps 1e-12 (:359-371)
    TT_DEVICE_CALL(ttmi_gemm(ctx_.raw(), wo, output->mutable_raw(), tokens, hidden, hidden, hidden, hidden, hidden, 1, 1.f, 0.f,
                             dt, Stream()));
    kernels::AddBiasLayerNormResidual(query_tensor, dense_bias_, layernorm_gamma_, layernorm_beta_, output, 1e-12f);
  } else {
    ttmi_epilogue_args args{};
    args.bias = dense_bias_.raw();
    args.residual = post_add_input ? query_tensor.raw() : nullptr;
    TT_DEVICE_CALL(ttmi_gemm_fused(ctx_.raw(), wo, output->mutable_raw(), tokens, hidden, hidden, hidden, hidden, hidden,
                                   post_add_input ? TTMI_EPI_BIAS_RESIDUAL : TTMI_EPI_BIAS, &args, dt, Stream()));
  }
}

void MultiHeadedAttention::operator()(const Tensor& key_tensor, const Tensor& value_tensor, const Tensor& query_tensor,
                                      const Tensor& attention_mask, const std::string& attn_type, Tensor* output,
                                      Tensor* att_score, std::unordered_map<std::string, Tensor*> layer_cache,
                                      bool pre_layernorm, bool post_layernorm, bool post_add_input,
                                      bool is_trans_weight) const {
  std::lock_guard<std::mutex> g(mutex_);
  TT_ENFORCE(attn_type == "self", "only attn_type \"self\" is built (\"context\" belongs to the decoder path)");
  TT_ENFORCE(layer_cache.empty(), "layer_cache belongs to the decoder path and is not built");
  TT_ENFORCE_EQ(query_tensor.n_dim(), (size_t)3, "The query_tensors should be a matrix with shape [batch_size, query_seq_len, hidden_size].");
  TT_ENFORCE(output != nullptr, "output must not be null");
  kernels::RequireGpu(query_tensor, "MultiHeadedAttention");
  MultiHeadedAttention::EnforceShapeAndType();
  (void)key_tensor;
  (void)value_tensor;

  const int64_t batch = query_tensor.shape(0), seq = query_tensor.shape(1), hidden = query_tensor.shape(2);
  TT_ENFORCE_EQ(hidden, dense_weight_.shape(0), "hidden size of the input and of the weights differ");
  TT_ENFORCE(core::SameDataType(query_tensor.dtype(), qkv_weight_.dtype()), "input and weights must share one element type");
  const int64_t heads = num_attention_heads_, d = hidden / heads;
  const int dt = kernels::DeviceDType(query_tensor);
  const DLDeviceType dev = query_tensor.device_type();
  const int dev_id = query_tensor.device_id();

  const Tensor* qkv_in = &query_tensor;
  if (pre_layernorm) {
    TT_ENFORCE(!layernorm_gamma_.is_null(), "pre_layernorm needs LayerNorm parameters");
    ln_query_.ReshapeAs(query_tensor.dtype(), {batch, seq, hidden}, dev, dev_id, "self/layernorm/Reshape");
    core::CopyBytes(ln_query_.mutable_raw(), dev, query_tensor.raw(), dev, (size_t)query_tensor.numel() * query_tensor.element_size());
    kernels::LayerNorm<float>(layernorm_gamma_, layernorm_beta_, &ln_query_, 1e-6f);
    qkv_in = &ln_query_;
  }

  // with the fused core V is kept transposed, [B,h,d,pitch]: its tiles are then plain copies
  const int64_t v_pitch = UseFusedCore(attention_mask, att_score, d, dt) ? RoundUp8(seq) : 0;
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
  TT_DEVICE_CALL(ttmi_gemm_fused(qkv_in->raw(), qkv_packed_.Get(qkv_weight_, is_trans_weight), nullptr, batch * seq, 3 * hidden,
                                 hidden, hidden, hidden, 3 * hidden, TTMI_EPI_QKV_SPLIT, &args, dt, Stream()));

  SelfAttentionTail(query_tensor, attention_mask, output, att_score, batch, seq, nullptr, v_pitch, post_layernorm,
                    post_add_input, is_trans_weight);
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
  const int64_t v_pitch = UseFusedCore(attention_mask, att_score, d, dt) ? RoundUp8(max_seq) : 0;
  Tensor* qkv[3] = {&q_, &k_, &v_};
  const char* names[3] = {"self/q/Reshape", "self/k/Reshape", "self/v/Reshape"};
  for (int i = 0; i < 3; ++i) {
    if (i == 2 && v_pitch > 0) qkv[i]->ReshapeAs(query_tensor.dtype(), {batch, heads, d, v_pitch}, dev, dev_id, names[i]);
    else qkv[i]->ReshapeAs(query_tensor.dtype(), {batch, heads, max_seq, d}, dev, dev_id, names[i]);
    if (v_pitch > 0) continue;
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
  args.v_seq_pitch = v_pitch;
  TT_DEVICE_CALL(ttmi_gemm_fused(query_tensor.raw(), qkv_packed_.Get(qkv_weight_, is_trans_weight), nullptr, plan.total,
                                 3 * hidden, hidden, hidden, hidden, 3 * hidden, TTMI_EPI_QKV_SPLIT_PAD, &args, dt, Stream()));

  SelfAttentionTail(query_tensor, attention_mask, output, att_score, batch, max_seq, &query_seq_len_list, v_pitch,
                    post_layernorm, post_add_input, is_trans_weight);
}

}  // namespace layers
}  // namespace turbo_transformers
