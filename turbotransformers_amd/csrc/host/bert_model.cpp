#include "bert_model.h"

#include <algorithm>
#include <cstring>

#include "core/device_context.h"
#include "loaders/npz_load.h"
#include "ttmi.h"

namespace turbo_transformers {

using core::Tensor;

static Tensor Take(BERTLayer::WeightMap* w, const std::string& name) {
  auto it = w->find(name);
  TT_ENFORCE(it != w->end(), "weight %s is missing", name.c_str());
  Tensor t = std::move(it->second);
  w->erase(it);
  return t;
}

BERTLayer::BERTLayer(WeightMap* w, const std::string& p, int64_t n_heads) {
  attention_.reset(new layers::BertAttention(Take(w, p + "attention.qkv.weight"), Take(w, p + "attention.qkv.bias"),
                                             Take(w, p + "attention.output.dense.weight"),
                                             Take(w, p + "attention.output.dense.bias"),
                                             Take(w, p + "attention.output.LayerNorm.weight"),
                                             Take(w, p + "attention.output.LayerNorm.bias"), n_heads));
  intermediate_.reset(new layers::BertIntermediate(Take(w, p + "intermediate.dense.weight"), Take(w, p + "intermediate.dense.bias")));
  output_.reset(new layers::BertOutput(Take(w, p + "output.dense.weight"), Take(w, p + "output.dense.bias"),
                                       Take(w, p + "output.LayerNorm.weight"), Take(w, p + "output.LayerNorm.bias")));
}

void BERTLayer::operator()(Tensor& hidden, Tensor& mask, Tensor* attention_out, Tensor* intermediate_out, Tensor* output) const {
  (*attention_)(hidden, mask, attention_out);
  (*intermediate_)(*attention_out, intermediate_out);
  (*output_)(*intermediate_out, *attention_out, output);
}

struct BertModel::Impl {
  Impl(WeightMap weights, DLDeviceType device_type, size_t n_layers, int64_t n_heads) {
    TT_ENFORCE(core::IsGpu(device_type), "this build runs on the GPU only");
    // host tensors -> device
    for (auto& kv : weights) {
      Tensor& t = kv.second;
      if (t.is_gpu()) continue;
      std::vector<int64_t> shape;
      for (size_t i = 0; i < t.n_dim(); ++i) shape.push_back(t.shape((int)i));
      Tensor dev(core::NewDLPackTensor(shape, t.dtype(), kDLROCM, 0, kv.first));
      core::CopyBytes(dev.mutable_raw(), kDLROCM, t.raw(), kDLCPU, (size_t)t.numel() * t.element_size());
      t = std::move(dev);
    }
    const std::string e = "embeddings.";
    embedding_.reset(new layers::BERTEmbedding(Take(&weights, e + "word_embeddings.weight"),
                                               Take(&weights, e + "position_embeddings.weight"),
                                               Take(&weights, e + "token_type_embeddings.weight"),
                                               Take(&weights, e + "LayerNorm.weight"), Take(&weights, e + "LayerNorm.bias")));
    for (size_t i = 0; i < n_layers; ++i) encoders_.emplace_back(&weights, "encoder.layer." + std::to_string(i) + ".", n_heads);
    if (weights.count("pooler.dense.weight"))
      pooler_.reset(new layers::BertPooler(Take(&weights, "pooler.dense.weight"), Take(&weights, "pooler.dense.bias")));
  }

  void Forward(const Tensor& ids, Tensor* mask, Tensor* seq_type, Tensor* position_ids, Tensor* hidden) {
    Tensor ext(nullptr);
    layers::PrepareBertMasks()(ids, mask, seq_type, position_ids, &ext);
    (*embedding_)(ids, *position_ids, *seq_type, hidden);
    for (auto& layer : encoders_) layer(*hidden, ext, &att_out_, &intermediate_out_, hidden);
  }

  std::unique_ptr<layers::BERTEmbedding> embedding_;
  std::vector<BERTLayer> encoders_;
  std::unique_ptr<layers::BertPooler> pooler_;
  Tensor att_out_{nullptr}, intermediate_out_{nullptr};  // reused by every layer and every call
};

static BertModel::WeightMap LoadNpzWeights(const std::string& filename) {
  BertModel::WeightMap out;
  for (auto& kv : loaders::LoadNpz(filename)) {
    const loaders::NpyArray& a = kv.second;
    DLDataType dt = a.kind == 'i' ? core::DataTypeTrait<int64_t>::v
                                  : (a.word_size == 4 ? core::DataTypeTrait<float>::v : core::DataTypeTrait<core::Half>::v);
    Tensor t(core::NewDLPackTensor(a.shape, dt, kDLCPU, 0, kv.first));
    std::memcpy(t.mutable_raw(), a.bytes.data(), a.bytes.size());
    out.emplace(kv.first, std::move(t));
  }
  return out;
}

BertModel::BertModel(const std::string& filename, DLDeviceType device_type, size_t n_layers, int64_t n_heads)
    : m_(new Impl(LoadNpzWeights(filename), device_type, n_layers, n_heads)) {}

BertModel::BertModel(WeightMap weights, DLDeviceType device_type, size_t n_layers, int64_t n_heads)
    : m_(new Impl(std::move(weights), device_type, n_layers, n_heads)) {}

BertModel::~BertModel() = default;

static void PadToDevice(const std::vector<std::vector<int64_t>>& rows, int64_t batch, int64_t width, Tensor* out) {
  std::vector<int64_t> host((size_t)(batch * width), 0);
  for (int64_t i = 0; i < batch; ++i) {
    TT_ENFORCE_LE((int64_t)rows[i].size(), width, "row longer than the padded width");
    std::copy(rows[i].begin(), rows[i].end(), host.begin() + i * width);
  }
  auto* p = out->Reshape<int64_t>({batch, width}, kDLROCM, 0, "BertModel/ids");
  core::CopyBytes(p, kDLROCM, host.data(), kDLCPU, host.size() * sizeof(int64_t));
}

std::vector<float> BertModel::operator()(const std::vector<std::vector<int64_t>>& inputs,
                                         const std::vector<std::vector<int64_t>>& position_ids,
                                         const std::vector<std::vector<int64_t>>& segment_ids, PoolType pooling,
                                         bool use_pooler) const {
  const int64_t batch = (int64_t)inputs.size();
  TT_ENFORCE_GT(batch, (int64_t)0, "empty batch");
  int64_t max_len = 0;
  for (auto& r : inputs) max_len = std::max<int64_t>(max_len, (int64_t)r.size());
  TT_ENFORCE_GT(max_len, (int64_t)0, "all inputs are empty");

  Tensor ids(nullptr), mask(nullptr), seq_type(nullptr), pos(nullptr);
  PadToDevice(inputs, batch, max_len, &ids);
  std::vector<std::vector<int64_t>> ones;
  for (auto& r : inputs) ones.emplace_back(r.size(), 1);
  PadToDevice(ones, batch, max_len, &mask);
  if (!position_ids.empty()) {
    TT_ENFORCE_EQ(position_ids.size(), (size_t)batch, "Position ids should have the same batch size as input ids");
    PadToDevice(position_ids, batch, max_len, &pos);
  }
  if (!segment_ids.empty()) {
    TT_ENFORCE_EQ(segment_ids.size(), (size_t)batch, "Segment ids should have the same batch size as input ids");
    PadToDevice(segment_ids, batch, max_len, &seq_type);
  }

  Tensor hidden(nullptr);
  m_->Forward(ids, &mask, &seq_type, &pos, &hidden);

  Tensor pooled(nullptr), projected(nullptr);
  const Tensor* result = &hidden;
  if (use_pooler) {
    TT_ENFORCE(m_->pooler_ != nullptr, "the weights hold no pooler");
    layers::kernels::SeqPool(hidden, pooling, &pooled);
    (*m_->pooler_)(pooled, &projected);
    result = &projected;
  }
  // hand back fp32 whatever the storage type of the model is
  std::vector<float> vec((size_t)result->numel());
  void* stream = core::DeviceContext::GetInstance().stream();
  if (core::ToDeviceDType(result->dtype()) == TTMI_F32) {
    core::CopyBytes(vec.data(), kDLCPU, result->raw(), kDLROCM, vec.size() * sizeof(float));
  } else {
    Tensor f32(core::NewDLPackTensorT<float>({result->numel()}, kDLROCM, 0, "BertModel/out"));
    TT_DEVICE_CALL(ttmi_convert(result->raw(), core::ToDeviceDType(result->dtype()), f32.mutable_raw(), TTMI_F32,
                                result->numel(), stream));
    core::CopyBytes(vec.data(), kDLCPU, f32.raw(), kDLROCM, vec.size() * sizeof(float));
  }
  core::DeviceContext::GetInstance().Wait();
  return vec;
}

void BertModel::Encode(const Tensor& input_ids, Tensor* hidden) const {
  Tensor mask(nullptr), seq_type(nullptr), pos(nullptr);
  m_->Forward(input_ids, &mask, &seq_type, &pos, hidden);
}

}  // namespace turbo_transformers
