#include "layers/quantized_layers.h"

#include <cmath>

#include "core/device_context.h"
#include "layers/kernels.h"
#include "ttmi.h"

namespace turbo_transformers {
namespace layers {

using core::DeviceContext;
using core::Tensor;

static void* Stream() { return DeviceContext::GetInstance().stream(); }

QuantizedLinear::QuantizedLinear(core::Tensor weight, core::Tensor bias, const std::string& activation)
    : weight_(std::move(weight)), bias_(std::move(bias)) {
  TT_ENFORCE_EQ(bias_.numel(), weight_.shape(1), "bias and weight shape mismatch");
  if (activation == "gelu") act_ = TTMI_ACT_GELU;
  else if (activation == "tanh") act_ = TTMI_ACT_TANH;
  else if (activation == "relu") act_ = TTMI_ACT_RELU;
  else TT_ENFORCE(activation.empty(), "unknown activation %s", activation.c_str());
}

void QuantizedLinear::Prepare() const {
  if (prepared_) return;
  kernels::RequireGpu(weight_, "QuantizedLinear");
  TT_ENFORCE_EQ(weight_.n_dim(), (size_t)2, "weight must be [in, out]");
  const int64_t k = weight_.shape(0), n = weight_.shape(1);
  const DLDeviceType dev = weight_.device_type();
  const int id = weight_.device_id();
  Tensor w_nk(nullptr);
  float* t = w_nk.Reshape<float>({n, k}, dev, id, "QuantizedLinear/w_nk");
  TT_DEVICE_CALL(ttmi_transpose_2d(weight_.data<float>(), t, k, n, TTMI_F32, Stream()));
  int8_t* q = q_weight_.Reshape<int8_t>({n, k}, dev, id, "QuantizedLinear/q_weight");
  float* s = w_scales_.Reshape<float>({n}, dev, id, "QuantizedLinear/w_scales");
  TT_DEVICE_CALL(ttmi_quantize_weight_rows_i8(t, q, s, n, k, Stream()));
  act_scale_.Reshape<float>({TTMI_QUANT_SCALE_FLOATS}, dev, id, "QuantizedLinear/act_scale");
  prepared_ = true;
}

void QuantizedLinear::operator()(const Tensor& input_tensor, Tensor* output_tensor) const {
  kernels::RequireGpu(input_tensor, "QuantizedLinear");
  Prepare();
  const int64_t k = weight_.shape(0), n = weight_.shape(1);
  TT_ENFORCE_EQ(input_tensor.shape(-1), k, "input width and weight rows differ");
  const int64_t m = input_tensor.numel() / k;
  const DLDeviceType dev = input_tensor.device_type();
  const int id = input_tensor.device_id();
  int8_t* qx = q_input_.Reshape<int8_t>({m, k}, dev, id, "QuantizedLinear/q_input");
  std::vector<int64_t> shape;
  for (size_t i = 0; i + 1 < input_tensor.n_dim(); ++i) shape.push_back(input_tensor.shape((int)i));
  shape.push_back(n);
  float* out = output_tensor->Reshape<float>(shape, dev, id, "QuantizedLinear/Reshape");
  float* scale = act_scale_.mutableData<float>();
  TT_DEVICE_CALL(ttmi_quantize_rows_i8(input_tensor.data<float>(), qx, scale, m, k, Stream()));
  // int8 GEMM with the dequantisation folded into its store: the int32 accumulators stay on chip
  TT_DEVICE_CALL(ttmi_gemm_i8_dequant(qx, q_weight_.data<int8_t>(), out, scale, w_scales_.data<float>(),
                                      bias_.is_null() ? nullptr : bias_.data<float>(), act_, m, n, k, k, k, n, Stream()));
}

void QuantizedBertAttention::operator()(const Tensor& input_tensor, const Tensor& attention_mask, Tensor* output,
                                        Tensor* attn) const {
  std::lock_guard<std::mutex> g(mutex_);
  kernels::RequireGpu(input_tensor, "QuantizedBertAttention");
  TT_ENFORCE_EQ(input_tensor.n_dim(), (size_t)3, "input should be [batch, seq, hidden]");
  const int64_t B = input_tensor.shape(0), S = input_tensor.shape(1), H = input_tensor.shape(2), d = H / heads_;
  const DLDeviceType dev = input_tensor.device_type();
  const int id = input_tensor.device_id();
  // QKV projection (int8) -> fp32 [B,S,3,H]; then the reference's unfused fp32 chain
  qkv_(input_tensor, &qkv_out_);
  qkv_out_.Reshape<float>({B, S, 3, H}, dev, id, "self/qkv_out1/Reshape");
  q_.Reshape<float>({B, heads_, S, d}, dev, id, "self/q/Reshape");
  k_.Reshape<float>({B, heads_, S, d}, dev, id, "self/k/Reshape");
  v_.Reshape<float>({B, heads_, S, d}, dev, id, "self/v/Reshape");
  kernels::SplitAddBiasTransposeForScore(qkv_out_, qkv_bias_, q_, k_, v_);
  Tensor* score = attn != nullptr ? attn : &score_scratch_;
  score->Reshape<float>({B, heads_, S, S}, dev, id, "batch_gemm3/Reshape");
  kernels::BatchMatMul(q_, false, k_, true, 1.0f / std::sqrt((float)d), score, 0.f);
  kernels::ApplyMaskAndSoftmax(score, attention_mask, 1.0f);
  ctx_.Reshape<float>({B, heads_, S, d}, dev, id, "ApplyMaskAndSoftmax/Reshape");
  kernels::BatchMatMul(*score, false, v_, false, 1.0f, &ctx_, 0.f);
  merged_.Reshape<float>({B, S, H}, dev, id, "batch_gemm4/Reshape");
  kernels::TransposeForScore(&merged_, ctx_);
  dense_(merged_, output);
  kernels::AddBiasLayerNorm<float>(input_tensor, dense_bias_, ln_weight_, ln_bias_, output, 1e-12f);
}

}  // namespace layers
}  // namespace turbo_transformers
