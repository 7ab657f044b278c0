#include "layers/bert_layers.h"

#include "core/device_context.h"
#include "ttmi.h"

namespace turbo_transformers {
namespace layers {

using core::DeviceContext;
using core::Tensor;

static void* Stream() { return DeviceContext::GetInstance().stream(); }

// ------------------------------------------------------------------------ embedding -----
void BERTEmbedding::EnforceShapeAndType() const {
  TT_ENFORCE_EQ(word_embedings_.n_dim(), (size_t)2, "word embeddings must be [vocab, hidden]");
  const int64_t hidden = word_embedings_.shape(1);
  TT_ENFORCE_EQ(position_embeddings_.shape(1), hidden, "position embedding width mismatch");
  TT_ENFORCE_EQ(token_type_embeddings_.shape(1), hidden, "token type embedding width mismatch");
  TT_ENFORCE_EQ(layer_norm_weights_.numel(), hidden, "LayerNorm weight size mismatch");
  TT_ENFORCE_EQ(layer_norm_bias_.numel(), hidden, "LayerNorm bias size mismatch");
}

void BERTEmbedding::operator()(const Tensor& input_ids, const Tensor& position_ids, const Tensor& token_type_ids,
                               Tensor* output_tensor) const {
  kernels::RequireGpu(input_ids, "BERTEmbedding");
  TT_ENFORCE_EQ(input_ids.n_dim(), (size_t)2, "The input ids should be a matrix.");
  TT_ENFORCE_EQ(position_ids.numel(), input_ids.numel(), "position_ids and input_ids differ in size");
  TT_ENFORCE_EQ(token_type_ids.numel(), input_ids.numel(), "token_type_ids and input_ids differ in size");
  const int64_t B = input_ids.shape(0), S = input_ids.shape(1), hidden = word_embedings_.shape(1);
  output_tensor->ReshapeAs(word_embedings_.dtype(), {B, S, hidden}, input_ids.device_type(), input_ids.device_id(),
                           "BERTEmbedding/Reshape");
  // three lookups + LayerNorm (bert_embedding.cpp:53-64) as one gather kernel
  if (kernels::KeepsFp32Residual(*output_tensor)) {
    core::Tensor* out32 = output_tensor->EnsureShadow();
    TT_DEVICE_CALL(ttmi_bert_embedding_residual32(
        output_tensor->mutable_raw(), out32->mutableData<float>(), input_ids.data<int64_t>(), position_ids.data<int64_t>(),
        token_type_ids.data<int64_t>(), word_embedings_.raw(), position_embeddings_.raw(), token_type_embeddings_.raw(),
        layer_norm_weights_.raw(), layer_norm_bias_.raw(), B * S, hidden, word_embedings_.shape(0),
        position_embeddings_.shape(0), token_type_embeddings_.shape(0), 1e-12f, kernels::DeviceDType(word_embedings_), Stream()));
    return;
  }
  TT_DEVICE_CALL(ttmi_bert_embedding(output_tensor->mutable_raw(), input_ids.data<int64_t>(), position_ids.data<int64_t>(),
                                     token_type_ids.data<int64_t>(), word_embedings_.raw(), position_embeddings_.raw(),
                                     token_type_embeddings_.raw(), layer_norm_weights_.raw(), layer_norm_bias_.raw(), B * S,
                                     hidden, word_embedings_.shape(0), position_embeddings_.shape(0),
                                     token_type_embeddings_.shape(0), 1e-12f, kernels::DeviceDType(word_embedings_), Stream()));
}

// ------------------------------------------------------------------------------ FFN -----
static void GemmBiasAct(const Tensor& in, const void* w_nk, int64_t n, const Tensor& bias, int act, Tensor* out) {
  const int64_t k = in.shape(-1), m = in.numel() / k;
  ttmi_epilogue_args args{};
  args.bias = bias.raw();
  args.act = act;
  TT_DEVICE_CALL(ttmi_gemm_fused(in.raw(), w_nk, out->mutable_raw(), m, n, k, k, k, n, TTMI_EPI_BIAS_ACT, &args,
                                 kernels::DeviceDType(in), Stream()));
}

static void GemmThenAddBiasLayerNorm(const Tensor& in, const void* w_nk, int64_t n, const Tensor& bias, const Tensor& residual,
                                     const Tensor& gamma, const Tensor& beta, Tensor* out) {
  kernels::GemmAddBiasLayerNorm(in, w_nk, n, residual, bias, gamma, beta, out, 1e-12f);
}

static std::vector<int64_t> WithLastDim(const Tensor& t, int64_t last) {
  std::vector<int64_t> shape;
  for (size_t i = 0; i + 1 < t.n_dim(); ++i) shape.push_back(t.shape((int)i));
  shape.push_back(last);
  return shape;
}

void BertIntermediate::EnforceShapeAndType() const {
  TT_ENFORCE_EQ(dense_weight_.n_dim(), (size_t)2, "dense_weight must be a matrix");
  TT_ENFORCE_EQ(dense_bias_.n_dim(), (size_t)1, "dense_bias must be a vector");
  TT_ENFORCE_EQ(dense_weight_.shape(1), dense_bias_.shape(0), "weight and bias shape mismatch %ld, %ld",
                (long)dense_weight_.shape(1), (long)dense_bias_.shape(0));
}

void BertIntermediate::operator()(const Tensor& input_tensor, Tensor* output_tensor) const {
  kernels::RequireGpu(input_tensor, "BertIntermediate");
  TT_ENFORCE_EQ(input_tensor.shape(-1), dense_weight_.shape(0), "input width and weight rows differ");
  const int64_t n = dense_weight_.shape(1);
  output_tensor->ReshapeAs(input_tensor.dtype(), WithLastDim(input_tensor, n), input_tensor.device_type(),
                           input_tensor.device_id(), "BertIntermediate/Reshape");
  GemmBiasAct(input_tensor, packed_.Get(dense_weight_, false), n, dense_bias_, TTMI_ACT_GELU, output_tensor);
}

void BertOutput::EnforceShapeAndType() const {
  TT_ENFORCE_EQ(dense_weight_.n_dim(), (size_t)2, "dense_weight must be a matrix");
  TT_ENFORCE_EQ(dense_weight_.shape(1), dense_bias_.numel(), "weight and bias shape mismatch");
  TT_ENFORCE_EQ(layer_norm_weight_.numel(), dense_bias_.numel(), "LayerNorm weight size mismatch");
  TT_ENFORCE_EQ(layer_norm_bias_.numel(), dense_bias_.numel(), "LayerNorm bias size mismatch");
}

void BertOutput::operator()(const Tensor& hidden_states, const Tensor& input_tensor, Tensor* output_tensor) const {
  kernels::RequireGpu(hidden_states, "BertOutput");
  TT_ENFORCE_EQ(hidden_states.shape(-1), dense_weight_.shape(0), "hidden_states width and weight rows differ");
  const int64_t n = dense_weight_.shape(1);
  // the reference names this buffer "BERTEmbedding/Reshape" so that its model-aware planner
  // aliases a layer's output with the next layer's input (bert_output.cpp:41-46)
  output_tensor->ReshapeAs(hidden_states.dtype(), WithLastDim(hidden_states, n), hidden_states.device_type(),
                           hidden_states.device_id(), "BERTEmbedding/Reshape");
  GemmThenAddBiasLayerNorm(hidden_states, packed_.Get(dense_weight_, false), n, dense_bias_, input_tensor, layer_norm_weight_,
                           layer_norm_bias_, output_tensor);
}

void AlbertLayer::operator()(const Tensor& input_tensor, Tensor* hidden_output, Tensor* output_tensor) const {
  kernels::RequireGpu(input_tensor, "AlbertLayer");
  const int64_t f = dense_weight_.shape(1), n = dense_output_weight_.shape(1);
  hidden_output->ReshapeAs(input_tensor.dtype(), WithLastDim(input_tensor, f), input_tensor.device_type(),
                           input_tensor.device_id(), "AlbertLayer/Reshape");
  GemmBiasAct(input_tensor, packed1_.Get(dense_weight_, false), f, dense_bias_, TTMI_ACT_GELU, hidden_output);
  output_tensor->ReshapeAs(input_tensor.dtype(), WithLastDim(input_tensor, n), input_tensor.device_type(),
                           input_tensor.device_id(), "AlbertLayer/Reshape");
  GemmThenAddBiasLayerNorm(*hidden_output, packed2_.Get(dense_output_weight_, false), n, dense_output_bias_, input_tensor,
                           layer_norm_weight_, layer_norm_bias_, output_tensor);
}

// --------------------------------------------------------------------------- masks ------
void PrepareBertMasks::operator()(const Tensor& inputs, Tensor* att_mask, Tensor* seq_type, Tensor* position_ids,
                                  Tensor* extended_attention_mask) const {
  kernels::RequireGpu(inputs, "PrepareBertMasks");
  TT_ENFORCE_EQ(inputs.n_dim(), (size_t)2, "inputs should be [batch, seq]");
  const int64_t B = inputs.shape(0), S = inputs.shape(1);
  const DLDeviceType dev = inputs.device_type();
  const int id = inputs.device_id();
  if (position_ids->is_null()) {
    auto* p = position_ids->Reshape<int64_t>({B, S}, dev, id, "PrepareBertMasks/possitionids/Reshape");
    kernels::common::Sequence(p, B, S, dev);
  }
  if (seq_type->is_null()) {
    auto* p = seq_type->Reshape<int64_t>({B, S}, dev, id, "PrepareBertMasks/seqids/Reshape");
    kernels::common::Fill<int64_t>(p, B * S, 0, dev);
  }
  if (att_mask->is_null()) {
    auto* p = att_mask->Reshape<int64_t>({B, S}, dev, id, "PrepareBertMasks/attmask/Reshape");
    kernels::common::Fill<int64_t>(p, B * S, 1, dev);
  }
  auto* ext = extended_attention_mask->Reshape<float>({att_mask->shape(0), 1, 1, att_mask->shape(1)}, dev, id,
                                                      "PrepareBertMasks/extendedattnmask/Reshape");
  kernels::common::Transform(att_mask->mutableData<int64_t>(), ext, att_mask->numel(), dev);
}

// -------------------------------------------------------------------------- pooling -----
SequencePool::SequencePool(const std::string& pool_type) {
  if (pool_type == "First") pool_type_ = kernels::PoolType::kFirst;
  else if (pool_type == "Last") pool_type_ = kernels::PoolType::kLast;
  else if (pool_type == "Mean") pool_type_ = kernels::PoolType::kMean;
  else if (pool_type == "Max") pool_type_ = kernels::PoolType::kMax;
  else TT_THROW("The input pool_type(%s) is not int ['First', 'Last', 'Mean', 'Max'].", pool_type.c_str());
}

void SequencePool::operator()(const Tensor& input, Tensor* output) const { kernels::SeqPool(input, pool_type_, output); }

static void CheckFfn(const Tensor& input, const Tensor& w1, const Tensor& b1, const Tensor& w2, const Tensor& b2, bool trans,
                     const char* who) {
  kernels::RequireGpu(input, who);
  TT_ENFORCE_EQ(input.n_dim(), (size_t)3, "input should be [batch_size, input_len, model_dim]");
  TT_ENFORCE(w1.n_dim() == 2 && w2.n_dim() == 2, "dense weights must be matrices");
  TT_ENFORCE_EQ(PackedWeight::InDim(w1, trans), input.shape(2), "dense weight and input tensor should have the same model_dim.");
  TT_ENFORCE_EQ(PackedWeight::InDim(w2, trans), PackedWeight::OutDim(w1, trans), "the two dense weights do not chain");
  TT_ENFORCE_EQ(PackedWeight::OutDim(w2, trans), input.shape(2), "the second dense weight must map back to model_dim");
  TT_ENFORCE_EQ(b1.numel(), PackedWeight::OutDim(w1, trans), "dense_bias_1 size mismatch");
  TT_ENFORCE_EQ(b2.numel(), input.shape(2), "dense_bias_2 size mismatch");
  TT_ENFORCE(core::SameDataType(input.dtype(), w1.dtype()), "input and weights must share one element type");
}

void PositionwiseFeedForward::operator()(const Tensor& input_tensor, Tensor* output, bool is_trans_weight) const {
  CheckFfn(input_tensor, dense_weight_1_, dense_bias_1_, dense_weight_2_, dense_bias_2_, is_trans_weight, "PositionwiseFeedForward");
  const int64_t model_dim = input_tensor.shape(2), d_ff = PackedWeight::OutDim(dense_weight_1_, is_trans_weight);
  const int64_t m = input_tensor.numel() / model_dim;
  const DLDeviceType dev = input_tensor.device_type();
  const int id = input_tensor.device_id();
  normed_.ReshapeAs(input_tensor.dtype(), {input_tensor.shape(0), input_tensor.shape(1), model_dim}, dev, id, "FFN/LayerNorm/Reshape");
  core::CopyBytes(normed_.mutable_raw(), dev, input_tensor.raw(), dev, (size_t)input_tensor.numel() * input_tensor.element_size());
  kernels::LayerNorm<float>(layer_norm_weight_, layer_norm_bias_, &normed_, 1e-12f);
  hidden_.ReshapeAs(input_tensor.dtype(), {m, d_ff}, dev, id, "FFN/gemm0/Reshape");
  GemmBiasAct(normed_, packed1_.Get(dense_weight_1_, is_trans_weight), d_ff, dense_bias_1_, TTMI_ACT_RELU, &hidden_);
  output->ReshapeAs(input_tensor.dtype(), {input_tensor.shape(0), input_tensor.shape(1), model_dim}, dev, id, "FFN/Reshape");
  // gemm1 + AddInputBias in one launch
  ttmi_epilogue_args args{};
  args.bias = dense_bias_2_.raw();
  args.residual = input_tensor.raw();
  TT_DEVICE_CALL(ttmi_gemm_fused(hidden_.raw(), packed2_.Get(dense_weight_2_, is_trans_weight), output->mutable_raw(), m, model_dim,
                                 d_ff, d_ff, d_ff, model_dim, TTMI_EPI_BIAS_RESIDUAL, &args, kernels::DeviceDType(input_tensor),
                                 Stream()));
}

void DistrillFFN::operator()(const Tensor& input_tensor, Tensor* output, bool is_trans_weight) const {
  CheckFfn(input_tensor, dense_weight_1_, dense_bias_1_, dense_weight_2_, dense_bias_2_, is_trans_weight, "DistrillFFN");
  const int64_t model_dim = input_tensor.shape(2), d_ff = PackedWeight::OutDim(dense_weight_1_, is_trans_weight);
  const int64_t m = input_tensor.numel() / model_dim;
  const DLDeviceType dev = input_tensor.device_type();
  const int id = input_tensor.device_id();
  hidden_.ReshapeAs(input_tensor.dtype(), {m, d_ff}, dev, id, "FFN/gemm0/Reshape");
  GemmBiasAct(input_tensor, packed1_.Get(dense_weight_1_, is_trans_weight), d_ff, dense_bias_1_, TTMI_ACT_GELU, &hidden_);
  output->ReshapeAs(input_tensor.dtype(), {input_tensor.shape(0), input_tensor.shape(1), model_dim}, dev, id, "FFN/Reshape");
  // gemm1, then AddInputBias + LayerNorm as one AddBiasLayerNorm
  GemmThenAddBiasLayerNorm(hidden_, packed2_.Get(dense_weight_2_, is_trans_weight), model_dim, dense_bias_2_, input_tensor,
                           layer_norm_weight_, layer_norm_bias_, output);
}

void BertPooler::operator()(const Tensor& input_tensor, Tensor* output_tensor) const {
  kernels::RequireGpu(input_tensor, "BertPooler");
  TT_ENFORCE_EQ(input_tensor.shape(-1), dense_weight_.shape(0), "input width and weight rows differ");
  const int64_t n = dense_weight_.shape(1);
  output_tensor->ReshapeAs(input_tensor.dtype(), WithLastDim(input_tensor, n), input_tensor.device_type(),
                           input_tensor.device_id(), "BertPooler/Reshape");
  GemmBiasAct(input_tensor, packed_.Get(dense_weight_, false), n, dense_bias_, TTMI_ACT_TANH, output_tensor);
}

void LinearBias::operator()(const Tensor& input_tensor, Tensor* output_tensor) const {
  kernels::RequireGpu(input_tensor, "LinearBias");
  TT_ENFORCE_EQ(input_tensor.shape(-1), weight_.shape(0), "input width and weight rows differ");
  const int64_t n = weight_.shape(1), k = weight_.shape(0), m = input_tensor.numel() / k;
  output_tensor->ReshapeAs(input_tensor.dtype(), WithLastDim(input_tensor, n), input_tensor.device_type(),
                           input_tensor.device_id(), "LinearBias/Reshape");
  ttmi_epilogue_args args{};
  args.bias = bias_.raw();
  TT_DEVICE_CALL(ttmi_gemm_fused(input_tensor.raw(), packed_.Get(weight_, false), output_tensor->mutable_raw(), m, n, k, k, k,
                                 n, TTMI_EPI_BIAS, &args, kernels::DeviceDType(input_tensor), Stream()));
}

// ----------------------------------------------------------------- stand-alone epilogues
void FusedAddBiasGELU::operator()(Tensor* output_tensor) const {
  kernels::AddBiasAct<float, kernels::ActivationType::Gelu>(dense_bias_, output_tensor);
}

void FusedAddBiasLayerNorm::operator()(const Tensor& input_tensor, Tensor* output_tensor) const {
  // (the quantized layers' epilogue: its result is what the next quantized Linear quantises)
  kernels::AddBiasLayerNormWithAbsmax(input_tensor, dense_bias_, layer_norm_weight_, layer_norm_bias_, output_tensor, 1e-12f);
}

}  // namespace layers
}  // namespace turbo_transformers
