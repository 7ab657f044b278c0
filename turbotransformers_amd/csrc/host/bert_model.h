// C++ model API of the reference's example (example/cpp/bert_model.h:26-41,
// example/cpp/bert_model.cpp:51-79): BertModel(npz file, device, layers, heads) whose
// operator() takes ragged id lists and returns the pooled vector, and BERTLayer =
// attention -> intermediate -> output on caller-owned temporaries.
//
// Weight names follow tools/convert_huggingface_bert_pytorch_to_npz.py:44-71:
//   embeddings.{word,position,token_type}_embeddings.weight, embeddings.LayerNorm.{weight,bias},
//   encoder.layer.N.attention.qkv.{weight,bias}, ...attention.output.dense.*, ...attention.output.LayerNorm.*,
//   ...intermediate.dense.*, ...output.dense.*, ...output.LayerNorm.*, pooler.dense.*
// with every dense weight stored [in, out].
#pragma once

#include <map>
#include <memory>
#include <string>
#include <vector>

#include "core/tensor.h"
#include "layers/bert_layers.h"
#include "layers/multi_headed_attention.h"

namespace turbo_transformers {

using PoolType = layers::kernels::PoolType;

struct BERTLayer {
  using WeightMap = std::map<std::string, core::Tensor>;
  // `prefix` is "encoder.layer.N."; the tensors are moved out of `weights`.
  BERTLayer(WeightMap* weights, const std::string& prefix, int64_t n_heads);

  void operator()(core::Tensor& hidden, core::Tensor& mask, core::Tensor* attention_out, core::Tensor* intermediate_out,
                  core::Tensor* output) const;

  std::unique_ptr<layers::BertAttention> attention_;
  std::unique_ptr<layers::BertIntermediate> intermediate_;
  std::unique_ptr<layers::BertOutput> output_;
};

class BertModel {
 public:
  using WeightMap = std::map<std::string, core::Tensor>;

  BertModel(const std::string& filename, DLDeviceType device_type, size_t n_layers, int64_t n_heads);
  // Same model from tensors already in memory (device tensors are used as they are, host
  // tensors are copied to the device).
  BertModel(WeightMap weights, DLDeviceType device_type, size_t n_layers, int64_t n_heads);
  ~BertModel();

  // Pads the ragged inputs to [B, max_len] with a 0/1 mask, runs embedding + encoder
  // (+ SequencePool, + pooler when use_pooler) and returns the pooled [B, H] vector.
  std::vector<float> operator()(const std::vector<std::vector<int64_t>>& inputs,
                                const std::vector<std::vector<int64_t>>& position_ids,
                                const std::vector<std::vector<int64_t>>& segment_ids, PoolType pooling = PoolType::kFirst,
                                bool use_pooler = false) const;

  // Device-resident forward: int64 ids [B,S] on the GPU -> last hidden state [B,S,H].
  void Encode(const core::Tensor& input_ids, core::Tensor* hidden) const;

 private:
  struct Impl;
  std::unique_ptr<Impl> m_;
};

}  // namespace turbo_transformers
