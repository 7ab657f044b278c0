#include "layers/packed_weight.h"

#include "core/device_context.h"
#include "layers/kernels.h"
#include "ttmi.h"

namespace turbo_transformers {
namespace layers {

const void* PackedWeight::Get(const core::Tensor& w, bool is_trans_weight) const {
  TT_ENFORCE_EQ(w.n_dim(), (size_t)2, "weights must be 2-D");
  kernels::RequireGpu(w, "weight");
  if (is_trans_weight) return w.raw();
  std::lock_guard<std::mutex> lock(mutex_);
  if (source_ != w.raw() || packed_.is_null()) {
    const int64_t K = w.shape(0), N = w.shape(1);
    packed_.ReshapeAs(w.dtype(), {N, K}, w.device_type(), w.device_id(), "PackedWeight");
    TT_DEVICE_CALL(ttmi_transpose_2d(w.raw(), packed_.mutable_raw(), K, N, core::ToDeviceDType(w.dtype()),
                                     core::DeviceContext::GetInstance().stream()));
    source_ = w.raw();
  }
  return packed_.raw();
}

}  // namespace layers
}  // namespace turbo_transformers
