#include "layers/kernels.h"

#include <algorithm>
#include <numeric>

#include "core/device_context.h"
#include "ttmi.h"

namespace turbo_transformers {
namespace layers {
namespace kernels {

using core::DeviceContext;
using core::Tensor;

static void* Stream() { return DeviceContext::GetInstance().stream(); }

void RequireGpu(const Tensor& t, const char* what) {
  if (!t.is_gpu()) TT_THROW("%s: tensor is not on the GPU; this build has no CPU kernels", what);
}

int DeviceDType(const Tensor& t) {
  const int dt = core::ToDeviceDType(t.dtype());
  TT_ENFORCE(dt == TTMI_F32 || dt == TTMI_F16 || dt == TTMI_BF16, "expected a float32/float16/bfloat16 tensor, got (%d,%d)",
             (int)t.dtype().code, (int)t.dtype().bits);
  return dt;
}

static void RequireSameDType(const Tensor& a, const Tensor& b, const char* what) {
  TT_ENFORCE(core::SameDataType(a.dtype(), b.dtype()), "%s: element types differ", what);
}

namespace common {
bool is_same_device_ctx(DLDevice a, DLDevice b) {
  return core::IsGpu(a.device_type) == core::IsGpu(b.device_type) && (a.device_type == kDLCPU) == (b.device_type == kDLCPU) &&
         a.device_id == b.device_id;
}
bool is_same_shape(const Tensor& a, const Tensor& b) {
  if (a.n_dim() != b.n_dim()) return false;
  for (size_t i = 0; i < a.n_dim(); ++i)
    if (a.shape((int)i) != b.shape((int)i)) return false;
  return true;
}
void Sequence(int64_t* data, int64_t rows, int64_t cols, DLDeviceType device) {
  TT_ENFORCE(core::IsGpu(device), "Sequence: device_type is not supported");
  TT_DEVICE_CALL(ttmi_sequence_rows_i64(data, rows, cols, Stream()));
}
template <>
void Fill<int64_t>(int64_t* data, int64_t size, int64_t val, DLDeviceType device) {
  TT_ENFORCE(core::IsGpu(device), "Fill: device_type is not supported");
  TT_DEVICE_CALL(ttmi_fill_i64(data, size, val, Stream()));
}
template <>
void Fill<float>(float* data, int64_t size, float val, DLDeviceType device) {
  TT_ENFORCE(core::IsGpu(device), "Fill: device_type is not supported");
  TT_DEVICE_CALL(ttmi_fill_f32(data, size, val, Stream()));
}
void Transform(int64_t* src_data, float* dst_data, int64_t size, DLDeviceType device) {
  TT_ENFORCE(core::IsGpu(device), "Transform: device_type is not supported");
  TT_DEVICE_CALL(ttmi_mask_transform(src_data, dst_data, size, Stream()));
}
}  // namespace common

void MatMul(const Tensor& A, bool a_trans, const Tensor& B, bool b_trans, float alpha, Tensor* out, float beta,
            const std::string) {
  TT_ENFORCE(!a_trans, "MatMul: a_trans is not used on the encoder path and is not built");
  RequireGpu(A, "MatMul");
  TT_ENFORCE(common::is_same_device_ctx(A.device_ctx(), B.device_ctx()), "MatMul error: the device of A and B is different.");
  TT_ENFORCE(common::is_same_device_ctx(A.device_ctx(), out->device_ctx()), "MatMul error: the device of A and out is different.");
  RequireSameDType(A, B, "MatMul");
  RequireSameDType(A, *out, "MatMul");
  const int64_t a_cols = A.shape(-1), a_rows = A.numel() / a_cols;
  const int64_t b_cols = B.shape(-1), b_rows = B.numel() / b_cols;
  const int64_t M = a_rows, N = b_trans ? b_rows : b_cols, K_a = a_cols, K_b = b_trans ? b_cols : b_rows;
  TT_ENFORCE_EQ(K_a, K_b, "matrix shape mismatch %ld vs %ld", (long)K_a, (long)K_b);
  TT_ENFORCE_EQ(out->numel(), M * N, "MatMul: output has the wrong size");
  TT_DEVICE_CALL(ttmi_gemm(A.raw(), B.raw(), out->mutable_raw(), M, N, K_a, K_a, b_trans ? K_a : N, N, b_trans ? 1 : 0,
                           alpha, beta, DeviceDType(A), Stream()));
}

void BatchMatMul(const Tensor& A, bool a_trans, const Tensor& B, bool b_trans, float alpha, Tensor* C, float beta,
                 const std::string) {
  TT_ENFORCE(!a_trans, "BatchMatMul: a_trans is not used on the encoder path and is not built");
  RequireGpu(A, "BatchMatMul");
  TT_ENFORCE_GT(A.n_dim(), (size_t)2, "A must at least be 3 dims");
  TT_ENFORCE_GT(B.n_dim(), (size_t)2, "B must at least be 3 dims");
  RequireSameDType(A, B, "BatchMatMul");
  RequireSameDType(A, *C, "BatchMatMul");
  const int64_t a_rows = A.shape(-2), a_cols = A.shape(-1), b_rows = B.shape(-2), b_cols = B.shape(-1);
  const int64_t a_batch = A.numel() / (a_rows * a_cols), b_batch = B.numel() / (b_rows * b_cols);
  TT_ENFORCE_EQ(a_batch, b_batch, "BatchSize mismatch");
  const int64_t M = a_rows, N = b_trans ? b_rows : b_cols, K_a = a_cols, K_b = b_trans ? b_cols : b_rows;
  TT_ENFORCE_EQ(K_a, K_b, "K mismatch");
  TT_ENFORCE_EQ(C->shape(-2), M, "C shape mismatch");
  TT_ENFORCE_EQ(C->shape(-1), N, "C shape mismatch");
  TT_ENFORCE_EQ(C->numel() / (M * N), b_batch, "C BatchSize mismatch");
  TT_DEVICE_CALL(ttmi_gemm_strided_batched(A.raw(), B.raw(), C->mutable_raw(), M, N, K_a, K_a, b_trans ? K_a : N, N,
                                           a_rows * a_cols, b_rows * b_cols, M * N, a_batch, b_trans ? 1 : 0, alpha, beta,
                                           DeviceDType(A), Stream()));
}

void SplitAddBiasTransposeForScore(const Tensor& input_tensor, const Tensor& bias_tensor, Tensor& q_out, Tensor& k_out,
                                   Tensor& v_out, const std::string) {
  RequireGpu(input_tensor, "SplitAddBiasTransposeForScore");
  TT_ENFORCE_EQ(input_tensor.n_dim(), (size_t)4, "input_tensor should be (batch_size, seq_length, 3, hidden)");
  TT_ENFORCE_EQ(input_tensor.shape(2), (int64_t)3, "the third dim of input_tensor should be 3");
  TT_ENFORCE_EQ(q_out.n_dim(), (size_t)4, "q_out should be (batch, heads, seq, size_per_head)");
  const int64_t B = q_out.shape(0), h = q_out.shape(1), S = q_out.shape(2), d = q_out.shape(3);
  TT_ENFORCE_EQ(input_tensor.shape(0) * input_tensor.shape(1), B * S, "batch*seq mismatch");
  TT_ENFORCE_EQ(input_tensor.shape(3), h * d, "hidden size mismatch");
  TT_ENFORCE_EQ(bias_tensor.numel(), 3 * h * d, "bias size mismatch");
  TT_ENFORCE(common::is_same_shape(q_out, k_out) && common::is_same_shape(q_out, v_out), "q/k/v shapes differ");
  TT_DEVICE_CALL(ttmi_split_add_bias_transpose_for_score(input_tensor.raw(), bias_tensor.raw(), q_out.mutable_raw(),
                                                         k_out.mutable_raw(), v_out.mutable_raw(), B, S, h, d,
                                                         DeviceDType(input_tensor), Stream()));
}

void SplitAddBiasTransposeForScorePad(const Tensor& input_tensor, const Tensor& bias_tensor, Tensor& q_out, Tensor& k_out,
                                      Tensor& v_out, const std::vector<int64_t>& seq_list, const std::string) {
  RequireGpu(input_tensor, "SplitAddBiasTransposeForScorePad");
  TT_ENFORCE_EQ(input_tensor.n_dim(), (size_t)4, "input_tensor should be (1, sum_seq_len, 3, hidden)");
  TT_ENFORCE_EQ(input_tensor.shape(0), (int64_t)1, "the first dim of a packed input should be 1");
  TT_ENFORCE_EQ(input_tensor.shape(2), (int64_t)3, "the third dim of input_tensor should be 3");
  auto plan = DeviceContext::GetInstance().GetSeqPlan(seq_list);
  const int64_t B = q_out.shape(0), h = q_out.shape(1), maxS = q_out.shape(2), d = q_out.shape(3);
  TT_ENFORCE_EQ(B, plan.batch, "batch size and seq_list length differ");
  TT_ENFORCE_EQ(maxS, plan.max_seq, "padded length and max(seq_list) differ");
  TT_ENFORCE_EQ(input_tensor.shape(1), plan.total, "packed length and sum(seq_list) differ");
  TT_ENFORCE_EQ(input_tensor.shape(3), h * d, "hidden size mismatch");
  TT_DEVICE_CALL(ttmi_split_add_bias_transpose_for_score_pad(input_tensor.raw(), bias_tensor.raw(), q_out.mutable_raw(),
                                                             k_out.mutable_raw(), v_out.mutable_raw(), plan.cu_seqlens, B,
                                                             maxS, h, d, DeviceDType(input_tensor), Stream()));
}

void TransposeForScore(Tensor* output, const Tensor& input, const std::string) {
  RequireGpu(input, "TransposeForScore");
  TT_ENFORCE_EQ(input.n_dim(), (size_t)4, "input should be a 4-D tensor");
  TT_ENFORCE_GE(output->n_dim(), (size_t)3, "output tensor dim should be greater than 3");
  TT_ENFORCE_EQ(input.numel(), output->numel(), "input.numel() and output.numel() should be the same");
  const int64_t B = input.shape(0), h = input.shape(1), S = input.shape(2), d = input.shape(3);
  TT_DEVICE_CALL(ttmi_transpose_for_score(input.raw(), output->mutable_raw(), B, S, h, d, DeviceDType(input), Stream()));
}

void TransposeForScorePad(Tensor* output, const Tensor& input, const std::vector<int64_t>& seq_list, const std::string) {
  RequireGpu(input, "TransposeForScorePad");
  TT_ENFORCE_EQ(input.n_dim(), (size_t)4, "input should be a 4-D tensor");
  auto plan = DeviceContext::GetInstance().GetSeqPlan(seq_list);
  const int64_t B = input.shape(0), h = input.shape(1), maxS = input.shape(2), d = input.shape(3);
  TT_ENFORCE_EQ(B, plan.batch, "batch size and seq_list length differ");
  TT_ENFORCE_EQ(maxS, plan.max_seq, "padded length and max(seq_list) differ");
  TT_ENFORCE_EQ(output->numel(), plan.total * h * d, "output size and sum(seq_list) differ");
  TT_DEVICE_CALL(ttmi_transpose_for_score_pad(input.raw(), output->mutable_raw(), plan.cu_seqlens, B, maxS, h, d,
                                              DeviceDType(input), Stream()));
}

void ApplyMaskAndSoftmax(Tensor* inout, const Tensor& att_mask, float scale, const std::string) {
  RequireGpu(*inout, "ApplyMaskAndSoftmax");
  TT_ENFORCE_EQ(inout->n_dim(), (size_t)4, "attention scores should be (batch, heads, from_len, to_len)");
  const int64_t B = inout->shape(0), h = inout->shape(1), F = inout->shape(2), T = inout->shape(3);
  bool is_2d = true;
  const float* mask = nullptr;
  if (!att_mask.is_null()) {
    // softmax.cpp:93-102: (B,T) / (B,1,T) / (B,1,1,T) broadcast over query rows, otherwise per row
    is_2d = att_mask.n_dim() == 2 || (att_mask.n_dim() == 3 && att_mask.shape(1) == 1) ||
            (att_mask.n_dim() == 4 && att_mask.shape(2) == 1);
    mask = att_mask.data<float>();
    TT_ENFORCE_EQ(att_mask.numel(), is_2d ? B * T : B * F * T, "attention mask has the wrong size");
  }
  TT_DEVICE_CALL(ttmi_apply_mask_and_softmax(inout->mutable_raw(), mask, B, h, F, T, is_2d ? 1 : 0, scale,
                                             DeviceDType(*inout), Stream()));
}

template <typename T>
void LayerNorm(const Tensor& gamma, const Tensor& beta, Tensor* out_tensor, T eps, const std::string) {
  RequireGpu(*out_tensor, "LayerNorm");
  const int64_t n = out_tensor->shape(-1), m = out_tensor->numel() / n;
  TT_ENFORCE_EQ(gamma.numel(), n, "LayerNorm gamma size mismatch");
  TT_ENFORCE_EQ(beta.numel(), n, "LayerNorm beta size mismatch");
  TT_DEVICE_CALL(ttmi_layer_norm(out_tensor->mutable_raw(), gamma.raw(), beta.raw(), m, n, (float)eps,
                                 DeviceDType(*out_tensor), Stream()));
}
template void LayerNorm<float>(const Tensor&, const Tensor&, Tensor*, float, const std::string);

template <typename T>
void AddBiasLayerNorm(const Tensor& input_tensor, const Tensor& bias_tensor, const Tensor& gamma_tensor,
                      const Tensor& beta_tensor, Tensor* out_tensor, T eps, const std::string) {
  RequireGpu(*out_tensor, "AddBiasLayerNorm");
  const int64_t n = input_tensor.shape(-1), m = input_tensor.numel() / n;
  TT_ENFORCE_EQ(n, gamma_tensor.shape(0), "AddBiasLayerNorm input_tensor.shape(-1) should be the same as gamma_tensor.shape(0)");
  TT_ENFORCE_EQ(n, beta_tensor.shape(0), "AddBiasLayerNorm input_tensor.shape(-1) should be the same as beta_tensor.shape(0)");
  TT_ENFORCE_EQ(n, bias_tensor.shape(0), "AddBiasLayerNorm input_tensor.shape(-1) should be the same as bias_tensor.shape(0)");
  TT_ENFORCE(common::is_same_shape(input_tensor, *out_tensor), "The shape of the input_tensor and out_tensor is not equal.");
  RequireSameDType(input_tensor, *out_tensor, "AddBiasLayerNorm");
  TT_DEVICE_CALL(ttmi_add_bias_layer_norm(out_tensor->mutable_raw(), input_tensor.raw(), bias_tensor.raw(), gamma_tensor.raw(),
                                          beta_tensor.raw(), m, n, (float)eps, DeviceDType(*out_tensor), Stream()));
}
template void AddBiasLayerNorm<float>(const Tensor&, const Tensor&, const Tensor&, const Tensor&, Tensor*, float,
                                      const std::string);

// AddBiasLayerNorm that also leaves the per-workgroup maxima of its result with the output tensor (fp32 tensors of
// the quantized layers: the next Linear quantises this result and needs max|x| for its scale).
void AddBiasLayerNormWithAbsmax(const Tensor& input_tensor, const Tensor& bias_tensor, const Tensor& gamma_tensor,
                                const Tensor& beta_tensor, Tensor* out_tensor, float eps) {
  RequireGpu(*out_tensor, "AddBiasLayerNorm");
  if (core::ToDeviceDType(out_tensor->dtype()) != TTMI_F32) {
    AddBiasLayerNorm<float>(input_tensor, bias_tensor, gamma_tensor, beta_tensor, out_tensor, eps);
    return;
  }
  const int64_t n = input_tensor.shape(-1), m = input_tensor.numel() / n;
  TT_ENFORCE_EQ(n, gamma_tensor.shape(0), "AddBiasLayerNorm input_tensor.shape(-1) should be the same as gamma_tensor.shape(0)");
  TT_ENFORCE_EQ(n, beta_tensor.shape(0), "AddBiasLayerNorm input_tensor.shape(-1) should be the same as beta_tensor.shape(0)");
  TT_ENFORCE_EQ(n, bias_tensor.shape(0), "AddBiasLayerNorm input_tensor.shape(-1) should be the same as bias_tensor.shape(0)");
  TT_ENFORCE(common::is_same_shape(input_tensor, *out_tensor), "The shape of the input_tensor and out_tensor is not equal.");
  RequireSameDType(input_tensor, *out_tensor, "AddBiasLayerNorm");
  void* out = out_tensor->mutable_raw();
  float* slots = out_tensor->EnsureAbsmax()->mutableData<float>();
  int written = 0;
  TT_DEVICE_CALL(ttmi_add_bias_layer_norm_absmax(out, input_tensor.raw(), bias_tensor.raw(), gamma_tensor.raw(), beta_tensor.raw(), m,
                                                 n, eps, TTMI_F32, slots, &written, Stream()));
  if (written == 0) out_tensor->DropAbsmax();
}

bool KeepsFp32Residual(const Tensor& t) { return core::ToDeviceDType(t.dtype()) == TTMI_BF16; }

void AddBiasLayerNormResidual(const Tensor& input_tensor, const Tensor& bias_tensor, const Tensor& gamma_tensor,
                              const Tensor& beta_tensor, Tensor* out_tensor, float eps) {
  if (!KeepsFp32Residual(*out_tensor)) {
    AddBiasLayerNorm<float>(input_tensor, bias_tensor, gamma_tensor, beta_tensor, out_tensor, eps);
    return;
  }
  RequireGpu(*out_tensor, "AddBiasLayerNorm");
  const int64_t n = input_tensor.shape(-1), m = input_tensor.numel() / n;
  TT_ENFORCE_EQ(n, gamma_tensor.shape(0), "AddBiasLayerNorm input_tensor.shape(-1) should be the same as gamma_tensor.shape(0)");
  TT_ENFORCE_EQ(n, beta_tensor.shape(0), "AddBiasLayerNorm input_tensor.shape(-1) should be the same as beta_tensor.shape(0)");
  TT_ENFORCE_EQ(n, bias_tensor.shape(0), "AddBiasLayerNorm input_tensor.shape(-1) should be the same as bias_tensor.shape(0)");
  TT_ENFORCE_EQ(input_tensor.numel(), out_tensor->numel(), "The shape of the input_tensor and out_tensor is not equal.");
  Tensor converted(nullptr);
  const float* residual = nullptr;
  if (input_tensor.shadow() != nullptr) {
    residual = input_tensor.shadow()->data<float>();
  } else {
    float* p = converted.Reshape<float>({m, n}, input_tensor.device_type(), input_tensor.device_id(), "residual32");
    TT_DEVICE_CALL(ttmi_convert(input_tensor.raw(), DeviceDType(input_tensor), p, TTMI_F32, m * n, Stream()));
    residual = p;
  }
  Tensor* out32 = out_tensor->EnsureShadow();
  TT_DEVICE_CALL(ttmi_add_bias_layer_norm_residual32(out_tensor->mutable_raw(), residual, bias_tensor.raw(), gamma_tensor.raw(),
                                                     beta_tensor.raw(), out32->mutableData<float>(), m, n, eps,
                                                     DeviceDType(*out_tensor), Stream()));
}

void GemmAddBiasLayerNorm(const Tensor& in, const void* w_nk, int64_t n, const Tensor& residual, const Tensor& bias_tensor,
                          const Tensor& gamma_tensor, const Tensor& beta_tensor, Tensor* out_tensor, float eps) {
  RequireGpu(*out_tensor, "AddBiasLayerNorm");
  const int64_t k = in.shape(-1), m = in.numel() / k;
  TT_ENFORCE_EQ(n, gamma_tensor.shape(0), "AddBiasLayerNorm input_tensor.shape(-1) should be the same as gamma_tensor.shape(0)");
  TT_ENFORCE_EQ(n, beta_tensor.shape(0), "AddBiasLayerNorm input_tensor.shape(-1) should be the same as beta_tensor.shape(0)");
  TT_ENFORCE_EQ(n, bias_tensor.shape(0), "AddBiasLayerNorm input_tensor.shape(-1) should be the same as bias_tensor.shape(0)");
  TT_ENFORCE_EQ(residual.numel(), m * n, "The shape of the input_tensor and out_tensor is not equal.");
  TT_ENFORCE_EQ(out_tensor->numel(), m * n, "The shape of the input_tensor and out_tensor is not equal.");
  const int dt = DeviceDType(*out_tensor);
  if (!KeepsFp32Residual(*out_tensor)) {
    TT_DEVICE_CALL(ttmi_gemm_bias_layer_norm(in.raw(), w_nk, out_tensor->mutable_raw(), residual.raw(), nullptr, bias_tensor.raw(),
                                             gamma_tensor.raw(), beta_tensor.raw(), nullptr, m, n, k, eps, dt, Stream()));
    return;
  }
  Tensor converted(nullptr);
  const float* residual32 = nullptr;
  if (residual.shadow() != nullptr) {
    residual32 = residual.shadow()->data<float>();
  } else {
    float* p = converted.Reshape<float>({m, n}, residual.device_type(), residual.device_id(), "residual32");
    TT_DEVICE_CALL(ttmi_convert(residual.raw(), DeviceDType(residual), p, TTMI_F32, m * n, Stream()));
    residual32 = p;
  }
  Tensor* out32 = out_tensor->EnsureShadow();
  TT_DEVICE_CALL(ttmi_gemm_bias_layer_norm(in.raw(), w_nk, out_tensor->mutable_raw(), nullptr, residual32, bias_tensor.raw(),
                                           gamma_tensor.raw(), beta_tensor.raw(), out32->mutableData<float>(), m, n, k, eps, dt,
                                           Stream()));
}

template <typename T, ActivationType ActType>
void AddBiasAct(const Tensor& bias, Tensor* out, const std::string) {
  RequireGpu(*out, "AddBiasAct");
  const int64_t n = out->shape(-1), m = out->numel() / n;
  TT_ENFORCE_EQ(n, bias.numel(), "AddBiasAct: bias size mismatch");
  TT_DEVICE_CALL(ttmi_add_bias_act(out->mutable_raw(), bias.raw(), m, n, (int)ActType, DeviceDType(*out), Stream()));
}
template void AddBiasAct<float, ActivationType::Gelu>(const Tensor&, Tensor*, const std::string);
template void AddBiasAct<float, ActivationType::Tanh>(const Tensor&, Tensor*, const std::string);
template void AddBiasAct<float, ActivationType::Relu>(const Tensor&, Tensor*, const std::string);

template <bool Add>
void LookupEmbedding(Tensor* out_tensor, const Tensor& embedding_table, const Tensor& ids_tensor, const std::string) {
  RequireGpu(*out_tensor, "LookupEmbedding");
  TT_ENFORCE_EQ(common::is_same_device_ctx(out_tensor->device_ctx(), embedding_table.device_ctx()), true,
                "The out_tensor and embedding_table should have the same device type and device id.");
  TT_ENFORCE_EQ(common::is_same_device_ctx(out_tensor->device_ctx(), ids_tensor.device_ctx()), true,
                "The out_tensor and ids_tensor should have the same device type and device id.");
  const int64_t num_ids = ids_tensor.numel(), hidden = embedding_table.shape(1), vocab = embedding_table.shape(0);
  TT_ENFORCE_EQ(out_tensor->numel(), num_ids * hidden, "LookupEmbedding: output size mismatch");
  TT_DEVICE_CALL(ttmi_lookup_embedding(out_tensor->mutable_raw(), embedding_table.raw(), ids_tensor.data<int64_t>(), num_ids,
                                       hidden, vocab, Add ? 1 : 0, DeviceDType(embedding_table), Stream()));
}
template void LookupEmbedding<true>(Tensor*, const Tensor&, const Tensor&, const std::string);
template void LookupEmbedding<false>(Tensor*, const Tensor&, const Tensor&, const std::string);

void SeqPool(const Tensor& input, PoolType pool_type, Tensor* output) {
  RequireGpu(input, "SeqPool");
  TT_ENFORCE_EQ(input.n_dim(), (size_t)3, "The input's dim should be 3, but the input's dim is %d", (int)input.n_dim());
  const int64_t B = input.shape(0), S = input.shape(1), H = input.shape(2);
  output->ReshapeAs(input.dtype(), {B, H}, input.device_type(), input.device_id(), "SeqPool/Reshape");
  TT_DEVICE_CALL(ttmi_seq_pool(input.raw(), output->mutable_raw(), B, S, H, (int)pool_type, DeviceDType(input), Stream()));
}

}  // namespace kernels
}  // namespace layers
}  // namespace turbo_transformers
