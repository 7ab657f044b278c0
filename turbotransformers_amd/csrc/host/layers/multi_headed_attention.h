// Attention layers of the encoder path, with the reference's class names and call
// signatures:
//   layers::MultiHeadedAttention            turbo_transformers/layers/multi_headed_attention.h:25-129
//   layers::BertAttention                   turbo_transformers/layers/bert_attention.h:25-47
//   layers::MultiHeadedAttentionSmartBatch  turbo_transformers/layers/multi_headed_attention_smart_batch.h:25-137
// MultiHeadedAttention also covers the decoder-side forms of the reference class: "context"
// attention over an encoder memory (separate q/k/v projections, memory_keys/memory_values cache),
// self attention with a growing self_keys/self_values cache, pre-LayerNorm and post_add_input.
//
// Device pipeline of one call (9 -> 6 launches by folding the memory-bound ops into GEMM
// epilogues):
//   QKV GEMM  + bias + head split            -> q,k,v [B,h,S,d]      (gemm012_fused + SplitAddBiasTranspose)
//   QK^T batched GEMM, alpha = 1/sqrt(d)     -> score [B,h,S,S]      (batch_gemm3)
//   mask + softmax in place                                           (ApplyMaskAndSoftmax)
//   P V batched GEMM storing [B,S,h,d]       -> ctx   [B,S,H]         (batch_gemm4 + TransposeForScore)
//   output GEMM                              -> out   [B,S,H]         (gemm5)
//   AddBiasLayerNorm(out, input) in place                             (AddBiasLayerNorm)
#pragma once

#include <mutex>
#include <string>
#include <unordered_map>
#include <vector>

#include "core/tensor.h"
#include "layers/packed_weight.h"

namespace turbo_transformers {
namespace layers {

class MultiHeadedAttention {
 public:
  MultiHeadedAttention(core::Tensor k_weight, core::Tensor k_bias, core::Tensor v_weight, core::Tensor v_bias,
                       core::Tensor q_weight, core::Tensor q_bias, core::Tensor dense_weight, core::Tensor dense_bias,
                       core::Tensor qkv_weight, core::Tensor qkv_bias, int64_t num_attention_heads)
      : k_weight_(std::move(k_weight)), k_bias_(std::move(k_bias)), v_weight_(std::move(v_weight)),
        v_bias_(std::move(v_bias)), q_weight_(std::move(q_weight)), q_bias_(std::move(q_bias)),
        dense_weight_(std::move(dense_weight)), dense_bias_(std::move(dense_bias)), qkv_weight_(std::move(qkv_weight)),
        qkv_bias_(std::move(qkv_bias)), layernorm_gamma_(nullptr), layernorm_beta_(nullptr),
        num_attention_heads_(num_attention_heads) {}

  MultiHeadedAttention(core::Tensor k_weight, core::Tensor k_bias, core::Tensor v_weight, core::Tensor v_bias,
                       core::Tensor q_weight, core::Tensor q_bias, core::Tensor dense_weight, core::Tensor dense_bias,
                       core::Tensor qkv_weight, core::Tensor qkv_bias, core::Tensor layernorm_gamma,
                       core::Tensor layernorm_beta, int64_t num_attention_heads)
      : k_weight_(std::move(k_weight)), k_bias_(std::move(k_bias)), v_weight_(std::move(v_weight)),
        v_bias_(std::move(v_bias)), q_weight_(std::move(q_weight)), q_bias_(std::move(q_bias)),
        dense_weight_(std::move(dense_weight)), dense_bias_(std::move(dense_bias)), qkv_weight_(std::move(qkv_weight)),
        qkv_bias_(std::move(qkv_bias)), layernorm_gamma_(std::move(layernorm_gamma)),
        layernorm_beta_(std::move(layernorm_beta)), num_attention_heads_(num_attention_heads) {}

  void EnforceShapeAndType() const;

  // query [B,F,H]; key/value [B,T,H] (read by "context" attention only); attention_mask additive fp32,
  // [B,1,1,T] / [B,1,T] (per key) or [B,F,T], or empty; output [B,F,H]; att_score [B,h,F,T] (may be
  // nullptr: then the probabilities stay internal).  layer_cache entries are [B,h,len,d] or empty.
  void operator()(const core::Tensor& key_tensor, const core::Tensor& value_tensor, const core::Tensor& query_tensor,
                  const core::Tensor& attention_mask, const std::string& attn_type, core::Tensor* output,
                  core::Tensor* att_score, std::unordered_map<std::string, core::Tensor*> layer_cache,
                  bool pre_layernorm = false, bool post_layernorm = false, bool post_add_input = false,
                  bool is_trans_weight = false) const;

  // The whole attention core runs as one kernel when nobody asks for the probabilities
  // (head size 64, additive key mask broadcast over the query rows).
  // batch, seq, heads: the shape of a dense batch (fp32 takes the fused kernel only for those, and only where it pays)
  static bool UseFusedCore(const core::Tensor& attention_mask, const core::Tensor* att_score, int64_t head_dim, int dtype,
                           int64_t batch = 0, int64_t seq = 0, int64_t heads = 0);

 protected:
  // Everything after q/k/v exist, shared by the dense and the smart-batch layers.
  // `fused_core`: the one-kernel attention core runs; `v_pitch` > 0: v holds V transposed, [B,h,d,v_pitch].
  // `seq` query positions against `key_seq` key positions held in k / v ([B,h,key_seq,d]).
  void AttentionTail(const core::Tensor& query_tensor, const core::Tensor& attention_mask, core::Tensor* output,
                     core::Tensor* att_score, int64_t batch, int64_t seq, int64_t key_seq, const core::Tensor& k,
                     const core::Tensor& v, const std::vector<int64_t>* seq_list, bool fused_core, int64_t v_pitch,
                     bool post_layernorm,
                     bool post_add_input, bool is_trans_weight) const;

  core::Tensor k_weight_, k_bias_, v_weight_, v_bias_, q_weight_, q_bias_;
  core::Tensor dense_weight_, dense_bias_, qkv_weight_, qkv_bias_;
  core::Tensor layernorm_gamma_, layernorm_beta_;
  int64_t num_attention_heads_;

  PackedWeight qkv_packed_, dense_packed_, q_packed_, k_packed_, v_packed_;
  // Per-call intermediates, reused across calls (Reshape keeps a buffer that is large enough).
  mutable core::Tensor q_, k_, v_, k_grown_, v_grown_, ctx_, score_scratch_, ln_query_;
  mutable std::mutex mutex_;  // the layer keeps per-call state, like the reference (…attention.cpp:32,272)
};

class BertAttention : public MultiHeadedAttention {
 public:
  BertAttention(core::Tensor qkv_weight, core::Tensor qkv_bias, core::Tensor dense_weight, core::Tensor dense_bias,
                core::Tensor layer_norm_weight, core::Tensor layer_norm_bias, int64_t num_attention_heads)
      : MultiHeadedAttention(core::Tensor(nullptr), core::Tensor(nullptr), core::Tensor(nullptr), core::Tensor(nullptr),
                             core::Tensor(nullptr), core::Tensor(nullptr), std::move(dense_weight), std::move(dense_bias),
                             std::move(qkv_weight), std::move(qkv_bias), std::move(layer_norm_weight),
                             std::move(layer_norm_bias), num_attention_heads) {
    EnforceShapeAndType();
  }
  void EnforceShapeAndType() const;

  void operator()(const core::Tensor& input_tensor, const core::Tensor& attention_mask, core::Tensor* output,
                  core::Tensor* attn = nullptr, bool is_trans_weight = false) const;
};

class MultiHeadedAttentionSmartBatch : public MultiHeadedAttention {
 public:
  using MultiHeadedAttention::MultiHeadedAttention;

  // query [1, sum(len), H] packed; attention_mask [B,1,max_len] (-1e9 on pad keys) or empty;
  // output [1, sum(len), H]; att_score [B,h,max_len,max_len] (padded).
  void operator()(const core::Tensor& key_tensor, const core::Tensor& value_tensor, const core::Tensor& query_tensor,
                  const core::Tensor& attention_mask, const std::string& attn_type, core::Tensor* output,
                  core::Tensor* att_score, std::unordered_map<std::string, core::Tensor*> layer_cache,
                  const std::vector<int64_t>& query_seq_len_list, const std::vector<int64_t>& key_seq_len_list,
                  bool pre_layernorm = false, bool post_layernorm = false, bool post_add_input = false,
                  bool is_trans_weight = false) const;
};

}  // namespace layers
}  // namespace turbo_transformers
