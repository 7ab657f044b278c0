#include "core/tensor.h"

#include <cstring>

#include "core/allocator.h"
#include "core/device_context.h"
#include "ttmi.h"

namespace turbo_transformers {
namespace core {

constexpr DLDataType DataTypeTrait<float>::v;
constexpr DLDataType DataTypeTrait<Half>::v;
constexpr DLDataType DataTypeTrait<BFloat16>::v;
constexpr DLDataType DataTypeTrait<int64_t>::v;
constexpr DLDataType DataTypeTrait<int32_t>::v;
constexpr DLDataType DataTypeTrait<int8_t>::v;

int ToDeviceDType(DLDataType t) {
  if (t.lanes != 1) return -1;
  if (t.code == kDLFloat && t.bits == 32) return TTMI_F32;
  if (t.code == kDLFloat && t.bits == 16) return TTMI_F16;
  if (t.code == kDLBfloat && t.bits == 16) return TTMI_BF16;
  if (t.code == kDLInt && t.bits == 8) return TTMI_I8;
  if (t.code == kDLInt && t.bits == 32) return TTMI_I32;
  if (t.code == kDLInt && t.bits == 64) return TTMI_I64;
  return -1;
}

namespace {

// An allocation made here: the DLManagedTensor, its shape storage and bookkeeping in one block.
struct OwnedBlock {
  DLManagedTensor managed;
  std::vector<int64_t> shape;
  size_t capacity_bytes = 0;
  std::string name;
};

void OwnedDeleter(DLManagedTensor* self) {
  auto* block = static_cast<OwnedBlock*>(self->manager_ctx);
  allocator::Allocator::GetInstance().free(self->dl_tensor.data, self->dl_tensor.device.device_type, block->name);
  delete block;
}

// Memory placed by the model-aware plan belongs to the plan (tensor.cpp:46-53 of the reference:
// DLManagedTensorDeletorWithoutData): only the descriptor is released.
void PlannedDeleter(DLManagedTensor* self) { delete static_cast<OwnedBlock*>(self->manager_ctx); }

int64_t Numel(const std::vector<int64_t>& shape) {
  return std::accumulate(shape.begin(), shape.end(), (int64_t)1, std::multiplies<int64_t>());
}

}  // namespace

DLManagedTensor* NewDLPackTensor(const std::vector<int64_t>& shape, DLDataType dtype, DLDeviceType device,
                                 int device_id, const std::string& name) {
  TT_ENFORCE(device == kDLCPU || IsGpu(device), "only cpu and gpu tensors are supported");
  for (int64_t d : shape) TT_ENFORCE_GE(d, (int64_t)0, "negative dimension");
  auto* block = new OwnedBlock();
  block->shape = shape;
  block->shape.reserve(8);
  block->name = name;
  block->capacity_bytes = (size_t)Numel(shape) * (dtype.bits / 8);
  DLTensor& t = block->managed.dl_tensor;
  auto& alloc = allocator::Allocator::GetInstance();
  const bool planned = IsGpu(device) && alloc.is_activation(name);
  try {
    t.data = alloc.allocate(block->capacity_bytes, device, name);
  } catch (...) {
    delete block;
    throw;
  }
  // Device memory made here is tagged kDLROCM: that is the tag torch on ROCm exports and accepts.
  t.device.device_type = IsGpu(device) ? kDLROCM : kDLCPU;
  t.device.device_id = device_id;
  t.ndim = (int32_t)block->shape.size();
  t.dtype = dtype;
  t.shape = block->shape.data();
  t.strides = nullptr;
  t.byte_offset = 0;
  block->managed.manager_ctx = block;
  block->managed.deleter = planned ? PlannedDeleter : OwnedDeleter;
  return &block->managed;
}

Tensor* Tensor::EnsureShadow() {
  const DLTensor& t = dl();
  std::vector<int64_t> shape(t.shape, t.shape + t.ndim);
  if (!shadow_) shadow_.reset(new Tensor(nullptr));
  shadow_->ReshapeAs(DataTypeTrait<float>::v, shape, t.device.device_type, t.device.device_id, "fp32_shadow");
  return shadow_.get();
}

Tensor* Tensor::EnsureAbsmax() {
  const DLTensor& t = dl();
  if (!absmax_) absmax_.reset(new Tensor(nullptr));
  absmax_->ReshapeAs(DataTypeTrait<float>::v, {TTMI_ABSMAX_SLOTS}, t.device.device_type, t.device.device_id, "absmax_slots");
  return absmax_.get();
}

void* Tensor::ReshapeAs(DLDataType dtype, const std::vector<int64_t>& shape_list, DLDeviceType device_type,
                        int device_id, const std::string& name) {
  shadow_.reset();  // new contents: a producer that wants an fp32 copy calls EnsureShadow() afterwards
  absmax_.reset();
  const size_t need = (size_t)Numel(shape_list) * (dtype.bits / 8);
  // Reuse only buffers allocated here (their shape storage and capacity are ours); tensors
  // imported from another framework are never resized in place.  A planned activation is looked up
  // again on every call: the plan may have changed, and a planned address must not be kept once
  // the schema is back to "naive".
  const bool planned = IsGpu(device_type) && allocator::Allocator::GetInstance().is_activation(name);
  if (!planned && managed_ != nullptr && managed_->deleter == OwnedDeleter) {
    auto* block = static_cast<OwnedBlock*>(managed_->manager_ctx);
    DLTensor& t = managed_->dl_tensor;
    const bool same_place = (IsGpu(t.device.device_type) == IsGpu(device_type)) &&
                            (t.device.device_type == kDLCPU) == (device_type == kDLCPU) &&
                            t.device.device_id == device_id;
    if (same_place && block->capacity_bytes >= need) {
      block->shape.assign(shape_list.begin(), shape_list.end());
      t.shape = block->shape.data();
      t.ndim = (int32_t)block->shape.size();
      t.dtype = dtype;
      return t.data;
    }
  }
  DLManagedTensor* fresh = NewDLPackTensor(shape_list, dtype, device_type, device_id, name);
  Release();
  managed_ = fresh;
  return managed_->dl_tensor.data;
}

Tensor Tensor::operator[](int64_t n) {
  const DLTensor& t = dl();
  TT_ENFORCE_GT(t.ndim, 1, "operator[] needs ndim > 1");
  TT_ENFORCE(n >= 0 && n < t.shape[0], "operator[] index out of range");
  Tensor r;
  r.is_view_ = true;
  r.view_shape_.assign(t.shape + 1, t.shape + t.ndim);
  const int64_t inner = Numel(r.view_shape_);
  r.view_.data = reinterpret_cast<char*>(t.data) + t.byte_offset + (uint64_t)(inner * n) * (t.dtype.bits / 8);
  r.view_.device = t.device;
  r.view_.ndim = t.ndim - 1;
  r.view_.dtype = t.dtype;
  r.view_.shape = r.view_shape_.data();
  r.view_.strides = nullptr;
  r.view_.byte_offset = 0;
  return r;
}

void CopyBytes(void* dst, DLDeviceType dst_dev, const void* src, DLDeviceType src_dev, size_t bytes) {
  if (bytes == 0) return;
  void* stream = DeviceContext::GetInstance().stream();
  if (dst_dev == kDLCPU && src_dev == kDLCPU) {
    std::memcpy(dst, src, bytes);
  } else if (dst_dev == kDLCPU) {
    TT_DEVICE_CALL(ttmi_memcpy(dst, src, bytes, TTMI_D2H, stream));
  } else if (src_dev == kDLCPU) {
    TT_DEVICE_CALL(ttmi_memcpy(dst, src, bytes, TTMI_H2D, stream));
  } else {
    TT_DEVICE_CALL(ttmi_memcpy_async(dst, src, bytes, TTMI_D2D, stream));
  }
}

}  // namespace core
}  // namespace turbo_transformers
