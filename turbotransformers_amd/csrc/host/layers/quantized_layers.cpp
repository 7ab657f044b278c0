#include "layers/quantized_layers.h"

#include <cmath>

#include "core/device_context.h"
#include "layers/kernels.h"
#include "layers/multi_headed_attention.h"
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
  std::lock_guard<std::mutex> lock(prepare_mutex_);
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

const int8_t* QuantizedLinear::QuantizeInput(const Tensor& input_tensor) const {
  kernels::RequireGpu(input_tensor, "QuantizedLinear");
  Prepare();
  const int64_t k = weight_.shape(0);
  TT_ENFORCE_EQ(input_tensor.shape(-1), k, "input width and weight rows differ");
  const int64_t m = input_tensor.numel() / k;
  int8_t* qx = q_input_.Reshape<int8_t>({m, k}, input_tensor.device_type(), input_tensor.device_id(), "QuantizedLinear/q_input");
  if (input_tensor.absmax() != nullptr) {
    // the kernel that produced the input left its per-workgroup maxima: one launch instead of two
    TT_DEVICE_CALL(ttmi_quantize_rows_i8_from_absmax(input_tensor.data<float>(), qx, act_scale_.mutableData<float>(),
                                                     input_tensor.absmax()->data<float>(), m, k, Stream()));
  } else {
    TT_DEVICE_CALL(ttmi_quantize_rows_i8(input_tensor.data<float>(), qx, act_scale_.mutableData<float>(), m, k, Stream()));
  }
  return qx;
}

void QuantizedLinear::operator()(const Tensor& input_tensor, Tensor* output_tensor) const {
  const int8_t* qx = QuantizeInput(input_tensor);
  const int64_t k = weight_.shape(0), n = weight_.shape(1), m = input_tensor.numel() / k;
  std::vector<int64_t> shape;
  for (size_t i = 0; i + 1 < input_tensor.n_dim(); ++i) shape.push_back(input_tensor.shape((int)i));
  shape.push_back(n);
  float* out = output_tensor->Reshape<float>(shape, input_tensor.device_type(), input_tensor.device_id(), "QuantizedLinear/Reshape");
  // int8 GEMM with the dequantisation folded into its store: the int32 accumulators stay on chip.  It also leaves the
  // per-workgroup maxima of its output with the tensor, for the Linear that quantises that output next.
  // (not for a bare product: that is the form in front of a fused bias + LayerNorm, which supplies its own)
  if (bias_.is_null() && act_ < 0) {
    TT_DEVICE_CALL(ttmi_gemm_i8_dequant(qx, q_weight_.data<int8_t>(), out, act_scale_.data<float>(), w_scales_.data<float>(), nullptr,
                                        act_, m, n, k, k, k, n, Stream()));
    return;
  }
  float* slots = output_tensor->EnsureAbsmax()->mutableData<float>();
  int written = 0;
  TT_DEVICE_CALL(ttmi_gemm_i8_dequant_absmax(qx, q_weight_.data<int8_t>(), out, act_scale_.data<float>(), w_scales_.data<float>(),
                                             bias_.is_null() ? nullptr : bias_.data<float>(), act_, m, n, k, k, k, n, slots,
                                             &written, Stream()));
  if (written == 0) output_tensor->DropAbsmax();
}

void QuantizedLinear::ProjectToHeads(const Tensor& input_tensor, const Tensor& bias, int64_t seq, int64_t heads, Tensor* q,
                                     Tensor* k_out, Tensor* v) const {
  TT_ENFORCE(bias_.is_null() && act_ < 0, "ProjectToHeads takes the bias as an argument");
  const int8_t* qx = QuantizeInput(input_tensor);
  const int64_t k = weight_.shape(0), n = weight_.shape(1), m = input_tensor.numel() / k;
  TT_ENFORCE_EQ(bias.numel(), n, "bias and weight shape mismatch");
  TT_ENFORCE(n % (3 * heads) == 0 && q->numel() == m * (n / 3), "q,k,v must be shaped [B, heads, S, d]");
  TT_DEVICE_CALL(ttmi_gemm_i8_dequant_qkv_split(qx, q_weight_.data<int8_t>(), act_scale_.data<float>(), w_scales_.data<float>(),
                                                bias.data<float>(), q->mutableData<float>(), k_out->mutableData<float>(),
                                                v->mutableData<float>(), m, n, k, k, k, seq, heads, n / (3 * heads), Stream()));
}

void QuantizedBertAttention::operator()(const Tensor& input_tensor, const Tensor& attention_mask, Tensor* output,
                                        Tensor* attn) const {
  std::lock_guard<std::mutex> g(mutex_);
  kernels::RequireGpu(input_tensor, "QuantizedBertAttention");
  TT_ENFORCE_EQ(input_tensor.n_dim(), (size_t)3, "input should be [batch, seq, hidden]");
  const int64_t B = input_tensor.shape(0), S = input_tensor.shape(1), H = input_tensor.shape(2), d = H / heads_;
  const DLDeviceType dev = input_tensor.device_type();
  const int id = input_tensor.device_id();
  // QKV projection (int8) with bias and head split in its store; then the reference's unfused fp32 chain
  q_.Reshape<float>({B, heads_, S, d}, dev, id, "self/q/Reshape");
  k_.Reshape<float>({B, heads_, S, d}, dev, id, "self/k/Reshape");
  v_.Reshape<float>({B, heads_, S, d}, dev, id, "self/v/Reshape");
  qkv_.ProjectToHeads(input_tensor, qkv_bias_, S, heads_, &q_, &k_, &v_);
  merged_.Reshape<float>({B, S, H}, dev, id, "batch_gemm4/Reshape");
  if (MultiHeadedAttention::UseFusedCore(attention_mask, attn, d, TTMI_F32, B, S, heads_)) {
    // nobody asked for the probabilities: the fp32 one-kernel attention (row-major V) in place of the four launches
    const float* mask = nullptr;
    if (!attention_mask.is_null()) {
      TT_ENFORCE_EQ(attention_mask.numel(), B * S, "attention mask has the wrong size");
      mask = attention_mask.data<float>();
    }
    // the kernel leaves the maxima of the context with the tensor: the output projection quantises it in one launch
    void* merged = merged_.mutable_raw();
    float* slots = merged_.EnsureAbsmax()->mutableData<float>();
    int written = 0;
    TT_DEVICE_CALL(ttmi_fused_attention_absmax(q_.raw(), k_.raw(), v_.raw(), mask, merged, nullptr, B, heads_, S, d, 0,
                                               1.0f / std::sqrt((float)d), TTMI_F32, slots, &written, Stream()));
    if (written == 0) merged_.DropAbsmax();
    dense_(merged_, output);
    kernels::AddBiasLayerNormWithAbsmax(input_tensor, dense_bias_, ln_weight_, ln_bias_, output, 1e-12f);
    return;
  }
  Tensor* score = attn != nullptr ? attn : &score_scratch_;
  score->Reshape<float>({B, heads_, S, S}, dev, id, "batch_gemm3/Reshape");
  kernels::BatchMatMul(q_, false, k_, true, 1.0f / std::sqrt((float)d), score, 0.f);
  kernels::ApplyMaskAndSoftmax(score, attention_mask, 1.0f);
  ctx_.Reshape<float>({B, heads_, S, d}, dev, id, "ApplyMaskAndSoftmax/Reshape");
  kernels::BatchMatMul(*score, false, v_, false, 1.0f, &ctx_, 0.f);
  kernels::TransposeForScore(&merged_, ctx_);
  dense_(merged_, output);
  kernels::AddBiasLayerNormWithAbsmax(input_tensor, dense_bias_, ln_weight_, ln_bias_, output, 1e-12f);
}

}  // namespace layers
}  // namespace turbo_transformers
