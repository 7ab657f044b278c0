// int8 Linear layers for the quantized BERT configuration: int8 weights with symmetric
// per-output-channel scales, int8 activations with one dynamic scale per call (max|x| over the
// whole [tokens, in] activation), int32 accumulation on v_mfma_i32_32x32x32_i8, fp32 dequant.
// Softmax and LayerNorm stay fp32.
//
// In the reference the int8 GEMM is not C++ at all: QBertIntermediate / QBertOutput wrap
// torch.quantization.quantize_dynamic modules (python/turbo_transformers/layers/qmodeling_bert.py:17,35)
// and only the fused fp32 epilogues are turbo kernels.  The classes here keep that split
// (QuantizedLinear alone has no bias; FusedAddBiasGELU / FusedAddBiasLayerNorm can follow it), let
// QuantizedLinear take the bias and activation into its own kernel, and add QuantizedBertAttention so
// that every Linear of the layer is int8.
#pragma once

#include <mutex>
#include <string>

#include "core/tensor.h"

namespace turbo_transformers {
namespace layers {

class QuantizedLinear {
 public:
  // weight: fp32 [in, out] (the layout every other layer takes); quantized on first use.
  explicit QuantizedLinear(core::Tensor weight) : weight_(std::move(weight)), bias_(nullptr) {}
  // With a bias and an activation ("gelu", "tanh", "relu", or "" for none) applied by the same kernel that
  // dequantises the product: Linear + FusedAddBiasGELU of QBertIntermediate as one call.
  QuantizedLinear(core::Tensor weight, core::Tensor bias, const std::string& activation);
  // output[tokens, out] (fp32) = act(dequant(q(input) * q(weight)^T) + bias)
  void operator()(const core::Tensor& input_tensor, core::Tensor* output_tensor) const;
  // A [hidden, 3*hidden] projection written as q,k,v[B, heads, S, d] = split(dequant(...) + bias): the Linear and
  // SplitAddBiasTransposeForScore of the attention in one kernel.  q,k,v are already shaped.
  void ProjectToHeads(const core::Tensor& input_tensor, const core::Tensor& bias, int64_t seq, int64_t heads, core::Tensor* q,
                      core::Tensor* k, core::Tensor* v) const;
  int64_t in_features() const { return weight_.shape(0); }
  int64_t out_features() const { return weight_.shape(1); }

 private:
  void Prepare() const;
  const int8_t* QuantizeInput(const core::Tensor& input_tensor) const;  // -> q_input_, scale in act_scale_
  core::Tensor weight_, bias_;
  int act_ = -1;  // ttmi_act; -1 = none
  mutable core::Tensor q_weight_, w_scales_, q_input_, act_scale_;
  mutable bool prepared_ = false;
  mutable std::mutex prepare_mutex_;  // the one-time weight quantisation; calls on one object are otherwise not concurrent
};

class QuantizedBertAttention {
 public:
  QuantizedBertAttention(core::Tensor qkv_weight, core::Tensor qkv_bias, core::Tensor dense_weight, core::Tensor dense_bias,
                         core::Tensor layer_norm_weight, core::Tensor layer_norm_bias, int64_t num_attention_heads)
      : qkv_(std::move(qkv_weight)), dense_(std::move(dense_weight)), qkv_bias_(std::move(qkv_bias)),
        dense_bias_(std::move(dense_bias)), ln_weight_(std::move(layer_norm_weight)), ln_bias_(std::move(layer_norm_bias)),
        heads_(num_attention_heads) {}
  // Same contract as BertAttention::operator() for fp32 tensors.
  void operator()(const core::Tensor& input_tensor, const core::Tensor& attention_mask, core::Tensor* output,
                  core::Tensor* attn = nullptr) const;

 private:
  QuantizedLinear qkv_, dense_;
  core::Tensor qkv_bias_, dense_bias_, ln_weight_, ln_bias_;
  int64_t heads_;
  mutable core::Tensor q_, k_, v_, ctx_, merged_, score_scratch_;
  mutable std::mutex mutex_;
};

}  // namespace layers
}  // namespace turbo_transformers
