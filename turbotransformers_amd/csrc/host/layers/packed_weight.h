// The MFMA GEMM kernels want every weight K-contiguous, i.e. [out, in] ("trans" layout),
// while the reference API hands layers [in, out] matrices unless is_trans_weight is set.
// PackedWeight produces the [out, in] form once, on the first call that needs it, and
// afterwards only returns the pointer.
#pragma once

#include <mutex>

#include "core/tensor.h"

namespace turbo_transformers {
namespace layers {

class PackedWeight {
 public:
  // Device pointer to W as [N, K]; `w` is [K, N] when !is_trans_weight, [N, K] otherwise.
  const void* Get(const core::Tensor& w, bool is_trans_weight) const;
  // Output width N of `w` under the given layout.
  static int64_t OutDim(const core::Tensor& w, bool is_trans_weight) { return is_trans_weight ? w.shape(0) : w.shape(1); }
  static int64_t InDim(const core::Tensor& w, bool is_trans_weight) { return is_trans_weight ? w.shape(1) : w.shape(0); }

 private:
  mutable std::mutex mutex_;  // two threads may make the first call of one layer object together
  mutable core::Tensor packed_;
  mutable const void* source_ = nullptr;
};

}  // namespace layers
}  // namespace turbo_transformers
