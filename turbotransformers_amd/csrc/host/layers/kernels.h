// Kernel API on core::Tensor, with the reference's names and argument meaning
// (turbo_transformers/layers/kernels/*.h).  Each function is the device branch only: it
// validates shapes on the host and enqueues one C-ABI call on the context stream.  CPU
// tensors are rejected -- this build is the MI355X path and has no CPU fallback.
//
//   reference header                       functions here
//   kernels/mat_mul.h                      MatMul, BatchMatMul
//   kernels/transpose.h                    SplitAddBiasTransposeForScore[Pad], TransposeForScore[Pad]
//   kernels/softmax.h                      ApplyMaskAndSoftmax
//   kernels/layer_norm.h                   LayerNorm, AddBiasLayerNorm
//   kernels/activation.h                   AddBiasAct
//   kernels/embedding.h                    LookupEmbedding
//   kernels/common.h (Sequence/Fill/Transform)   common::*
//   kernels/seq_pool.h                     SeqPool
#pragma once

#include <string>
#include <vector>

#include "core/tensor.h"

namespace turbo_transformers {
namespace layers {
namespace kernels {

enum class ActivationType { Gelu = 0, Tanh = 1, Relu = 2 };
enum class PoolType { kMax = 0, kMean, kFirst, kLast };

// out = alpha * A * op(B) + beta * out; A is viewed as [numel/last, last]  (mat_mul.cpp:30-118)
void MatMul(const core::Tensor& A, bool a_trans, const core::Tensor& B, bool b_trans, float alpha,
            core::Tensor* out, float beta, const std::string name = "MatMul");
// Strided-batched over all leading dims  (mat_mul.cpp:119-213)
void BatchMatMul(const core::Tensor& A, bool a_trans, const core::Tensor& B, bool b_trans, float alpha,
                 core::Tensor* C, float beta, const std::string name = "BatchMatMul");

// [B,S,3,h,d] + bias -> q,k,v [B,h,S,d]  (transpose.cpp:310-406)
void SplitAddBiasTransposeForScore(const core::Tensor& input_tensor, const core::Tensor& bias_tensor,
                                   core::Tensor& q_out, core::Tensor& k_out, core::Tensor& v_out,
                                   const std::string name = "SplitAddBiasTransposeForScore");
// packed [1,sum,3,h,d] -> zero-padded [B,h,maxS,d]  (transpose.cpp:459-580)
void SplitAddBiasTransposeForScorePad(const core::Tensor& input_tensor, const core::Tensor& bias_tensor,
                                      core::Tensor& q_out, core::Tensor& k_out, core::Tensor& v_out,
                                      const std::vector<int64_t>& seq_list,
                                      const std::string name = "SplitAddBiasTransposeForScorePad");
// [B,h,S,d] -> [B,S,h,d]  (transpose.cpp:158-191)
void TransposeForScore(core::Tensor* output, const core::Tensor& input, const std::string name = "TransposeForScore");
// [B,h,maxS,d] -> packed [1,sum,h*d]  (transpose.cpp:589-623)
void TransposeForScorePad(core::Tensor* output, const core::Tensor& input, const std::vector<int64_t>& seq_list,
                          const std::string name = "TransposeForScorePad");

// in place softmax(inout*scale + mask) over the last dim  (softmax.cpp:83-125)
void ApplyMaskAndSoftmax(core::Tensor* inout, const core::Tensor& att_mask, float scale,
                         const std::string name = "ApplyMaskAndSoftmax");

template <typename T>
void LayerNorm(const core::Tensor& gamma, const core::Tensor& beta, core::Tensor* out_tensor, T eps = 1e-12,
               const std::string name = "LayerNorm");
template <typename T>
void AddBiasLayerNorm(const core::Tensor& input_tensor, const core::Tensor& bias_tensor, const core::Tensor& gamma_tensor,
                      const core::Tensor& beta_tensor, core::Tensor* out_tensor, T eps = 1e-12,
                      const std::string name = "AddBiasLayerNorm");

template <typename T, ActivationType ActType>
void AddBiasAct(const core::Tensor& bias, core::Tensor* out, const std::string name = "AddBiasAct");

template <bool Add = false>
void LookupEmbedding(core::Tensor* out_tensor, const core::Tensor& embedding_table, const core::Tensor& ids_tensor,
                     const std::string name = "LookupEmbedding");

void SeqPool(const core::Tensor& input, PoolType pool_type, core::Tensor* output);

namespace common {
bool is_same_device_ctx(DLDevice a, DLDevice b);
bool is_same_shape(const core::Tensor& a, const core::Tensor& b);
void Sequence(int64_t* data, int64_t rows, int64_t cols, DLDeviceType device);  // data[r,c] = c
template <typename T>
void Fill(T* data, int64_t size, T val, DLDeviceType device);
void Transform(int64_t* src_data, float* dst_data, int64_t size, DLDeviceType device);  // -10000*(1-v)
}  // namespace common

// AddBiasLayerNorm as the layers call it.  fp32 / fp16: the plain kernel.  bfloat16: the residual
// is taken from input_tensor's fp32 shadow (or converted once if it has none), and the
// unrounded result is attached to out_tensor as its shadow, so a stack of layers keeps an fp32
// residual stream and rounds only GEMM operands.
void AddBiasLayerNormResidual(const core::Tensor& input_tensor, const core::Tensor& bias_tensor,
                              const core::Tensor& gamma_tensor, const core::Tensor& beta_tensor, core::Tensor* out_tensor,
                              float eps = 1e-12f);
void AddBiasLayerNormWithAbsmax(const core::Tensor& input_tensor, const core::Tensor& bias_tensor, const core::Tensor& gamma_tensor,
                                const core::Tensor& beta_tensor, core::Tensor* out_tensor, float eps);
bool KeepsFp32Residual(const core::Tensor& t);  // true for bfloat16 tensors
// out = AddBiasLayerNorm(in . w^T, residual) with the same treatment of the residual; `w_nk` is the
// [n, k] weight on the device, `out_tensor` already has its [.., n] shape.
void GemmAddBiasLayerNorm(const core::Tensor& in, const void* w_nk, int64_t n, const core::Tensor& residual,
                          const core::Tensor& bias_tensor, const core::Tensor& gamma_tensor, const core::Tensor& beta_tensor,
                          core::Tensor* out_tensor, float eps = 1e-12f);

// ---- fused forms used by the layers (no counterpart in the reference's kernel API) --------
int DeviceDType(const core::Tensor& t);  // ttmi_dtype of a floating tensor, throws otherwise
void RequireGpu(const core::Tensor& t, const char* what);

}  // namespace kernels
}  // namespace layers
}  // namespace turbo_transformers
