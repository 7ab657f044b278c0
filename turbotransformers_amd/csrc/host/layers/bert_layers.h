// The remaining layer objects of the BERT encoder path, with the reference's names and
// operator() signatures:
//   BERTEmbedding          turbo_transformers/layers/bert_embedding.h:23-52
//   BertIntermediate       turbo_transformers/layers/bert_intermediate.h
//   BertOutput             turbo_transformers/layers/bert_output.h
//   AlbertLayer            turbo_transformers/layers/albert_layer.h
//   PrepareBertMasks       turbo_transformers/layers/prepare_bert_masks.h
//   SequencePool           turbo_transformers/layers/sequence_pool.h
//   BertPooler             turbo_transformers/layers/bert_pooler.h
//   FusedAddBiasGELU       turbo_transformers/layers/addbias_act.h
//   FusedAddBiasLayerNorm  turbo_transformers/layers/addbias_layernorm.h
// Constructors take weights by value (callers move them in); operator() is const and
// allocates its output through Tensor::Reshape.
#pragma once

#include <string>

#include "core/tensor.h"
#include "layers/kernels.h"
#include "layers/packed_weight.h"

namespace turbo_transformers {
namespace layers {

class BERTEmbedding {
 public:
  BERTEmbedding(core::Tensor word_embeddings, core::Tensor position_embeddings, core::Tensor token_type_embeddings,
                core::Tensor layer_norm_weights, core::Tensor layer_norm_bias)
      : word_embedings_(std::move(word_embeddings)), position_embeddings_(std::move(position_embeddings)),
        token_type_embeddings_(std::move(token_type_embeddings)), layer_norm_weights_(std::move(layer_norm_weights)),
        layer_norm_bias_(std::move(layer_norm_bias)) {
    EnforceShapeAndType();
  }
  void EnforceShapeAndType() const;
  // ids / position_ids / token_type_ids: int64 [B,S]; output [B,S,H]
  void operator()(const core::Tensor& input_ids, const core::Tensor& position_ids, const core::Tensor& token_type_ids,
                  core::Tensor* output_tensor) const;

 private:
  core::Tensor word_embedings_, position_embeddings_, token_type_embeddings_, layer_norm_weights_, layer_norm_bias_;
};

class BertIntermediate {
 public:
  BertIntermediate(core::Tensor dense_weight, core::Tensor dense_bias)
      : dense_weight_(std::move(dense_weight)), dense_bias_(std::move(dense_bias)) {
    EnforceShapeAndType();
  }
  void EnforceShapeAndType() const;
  // output = gelu(input * W + b)   (bert_intermediate.cpp:32-50)
  void operator()(const core::Tensor& input_tensor, core::Tensor* output_tensor) const;

 private:
  core::Tensor dense_weight_, dense_bias_;
  PackedWeight packed_;
};

class BertOutput {
 public:
  BertOutput(core::Tensor dense_weight, core::Tensor dense_bias, core::Tensor layer_norm_weight, core::Tensor layer_norm_bias)
      : dense_weight_(std::move(dense_weight)), dense_bias_(std::move(dense_bias)),
        layer_norm_weight_(std::move(layer_norm_weight)), layer_norm_bias_(std::move(layer_norm_bias)) {
    EnforceShapeAndType();
  }
  void EnforceShapeAndType() const;
  // output = LN(hidden_states * W + b + input_tensor)   (bert_output.cpp:29-55)
  void operator()(const core::Tensor& hidden_states, const core::Tensor& input_tensor, core::Tensor* output_tensor) const;

 private:
  core::Tensor dense_weight_, dense_bias_, layer_norm_weight_, layer_norm_bias_;
  PackedWeight packed_;
};

class AlbertLayer {
 public:
  AlbertLayer(core::Tensor dense_weight, core::Tensor dense_bias, core::Tensor dense_output_weight,
              core::Tensor dense_output_bias, core::Tensor layer_norm_weight, core::Tensor layer_norm_bias)
      : dense_weight_(std::move(dense_weight)), dense_bias_(std::move(dense_bias)),
        dense_output_weight_(std::move(dense_output_weight)), dense_output_bias_(std::move(dense_output_bias)),
        layer_norm_weight_(std::move(layer_norm_weight)), layer_norm_bias_(std::move(layer_norm_bias)) {}
  // hidden_output = gelu(input W1 + b1); output = LN(hidden_output W2 + b2 + input)   (albert_layer.cpp:31-50)
  void operator()(const core::Tensor& input_tensor, core::Tensor* hidden_output, core::Tensor* output_tensor) const;

 private:
  core::Tensor dense_weight_, dense_bias_, dense_output_weight_, dense_output_bias_, layer_norm_weight_, layer_norm_bias_;
  PackedWeight packed1_, packed2_;
};

// Feed-forward blocks of the decoder / DistilBERT wrappers (positionwise_ffn.h:23-84).  Weights are
// [in, out], or [out, in] when called with is_trans_weight.
class PositionwiseFeedForward {
 public:
  PositionwiseFeedForward(core::Tensor dense_weight_1, core::Tensor dense_bias_1, core::Tensor dense_weight_2,
                          core::Tensor dense_bias_2, core::Tensor layer_norm_weight, core::Tensor layer_norm_bias)
      : dense_weight_1_(std::move(dense_weight_1)), dense_bias_1_(std::move(dense_bias_1)),
        dense_weight_2_(std::move(dense_weight_2)), dense_bias_2_(std::move(dense_bias_2)),
        layer_norm_weight_(std::move(layer_norm_weight)), layer_norm_bias_(std::move(layer_norm_bias)) {}
  // output = input + relu(LN(input) W1 + b1) W2 + b2, LayerNorm eps 1e-12   (positionwise_ffn.cpp:33-77)
  void operator()(const core::Tensor& input_tensor, core::Tensor* output, bool is_trans_weight = false) const;

 private:
  core::Tensor dense_weight_1_, dense_bias_1_, dense_weight_2_, dense_bias_2_, layer_norm_weight_, layer_norm_bias_;
  PackedWeight packed1_, packed2_;
  mutable core::Tensor normed_, hidden_;
};

class DistrillFFN {
 public:
  DistrillFFN(core::Tensor dense_weight_1, core::Tensor dense_bias_1, core::Tensor dense_weight_2, core::Tensor dense_bias_2,
              core::Tensor layer_norm_weight, core::Tensor layer_norm_bias)
      : dense_weight_1_(std::move(dense_weight_1)), dense_bias_1_(std::move(dense_bias_1)),
        dense_weight_2_(std::move(dense_weight_2)), dense_bias_2_(std::move(dense_bias_2)),
        layer_norm_weight_(std::move(layer_norm_weight)), layer_norm_bias_(std::move(layer_norm_bias)) {}
  // output = LN(input + gelu(input W1 + b1) W2 + b2), eps 1e-12   (positionwise_ffn.cpp:79-127)
  void operator()(const core::Tensor& input_tensor, core::Tensor* output, bool is_trans_weight = false) const;

 private:
  core::Tensor dense_weight_1_, dense_bias_1_, dense_weight_2_, dense_bias_2_, layer_norm_weight_, layer_norm_bias_;
  PackedWeight packed1_, packed2_;
  mutable core::Tensor hidden_;
};

class PrepareBertMasks {
 public:
  // Fills missing position ids (0..S-1), token types (0) and mask (1), and builds the additive
  // mask -10000*(1-mask) as fp32 [B,1,1,S]   (prepare_bert_masks.cpp:24-66)
  void operator()(const core::Tensor& inputs, core::Tensor* att_mask, core::Tensor* seq_type, core::Tensor* position_ids,
                  core::Tensor* extended_attention_mask) const;
};

class SequencePool {
 public:
  explicit SequencePool(const std::string& pool_type);
  void operator()(const core::Tensor& input, core::Tensor* output) const;  // [B,S,H] -> [B,H]

 private:
  kernels::PoolType pool_type_;
};

class BertPooler {
 public:
  BertPooler(core::Tensor dense_weight, core::Tensor dense_bias)
      : dense_weight_(std::move(dense_weight)), dense_bias_(std::move(dense_bias)) {}
  // output = tanh(input * W + b)   (bert_pooler.cpp:25-37)
  void operator()(const core::Tensor& input_tensor, core::Tensor* output_tensor) const;

 private:
  core::Tensor dense_weight_, dense_bias_;
  PackedWeight packed_;
};

// output = input * W + b on the MFMA GEMM with a bias epilogue.  No counterpart among the
// reference's C++ layers: its ALBERT wrapper calls a torch nn.Linear for the embedding
// projection (python layers/modeling_albert.py:254); this keeps that GEMM on the work stream.
class LinearBias {
 public:
  LinearBias(core::Tensor weight, core::Tensor bias) : weight_(std::move(weight)), bias_(std::move(bias)) {}
  void operator()(const core::Tensor& input_tensor, core::Tensor* output_tensor) const;

 private:
  core::Tensor weight_, bias_;  // weight [in, out]
  PackedWeight packed_;
};

class FusedAddBiasGELU {
 public:
  explicit FusedAddBiasGELU(core::Tensor dense_bias) : dense_bias_(std::move(dense_bias)) {}
  void operator()(core::Tensor* output_tensor) const;  // in place (addbias_act.cpp:20-23)

 private:
  core::Tensor dense_bias_;
};

class FusedAddBiasLayerNorm {
 public:
  FusedAddBiasLayerNorm(core::Tensor dense_bias, core::Tensor layer_norm_weight, core::Tensor layer_norm_bias)
      : dense_bias_(std::move(dense_bias)), layer_norm_weight_(std::move(layer_norm_weight)),
        layer_norm_bias_(std::move(layer_norm_bias)) {}
  // output = LN(output + input + bias) in place (addbias_layernorm.cpp:20-24)
  void operator()(const core::Tensor& input_tensor, core::Tensor* output_tensor) const;

 private:
  core::Tensor dense_bias_, layer_norm_weight_, layer_norm_bias_;
};

}  // namespace layers
}  // namespace turbo_transformers
