// core::Tensor: a DLPack payload that is empty, owns a DLManagedTensor, or is a non-owning
// view (result of operator[]).  Mirrors the reference's interface
// (turbo_transformers/core/tensor.h:117-354): from/to DLPack with ownership transfer,
// shape(i) with negative indices, Reshape<T>(shape, device, id, name) that keeps the buffer
// when it is large enough, data<T>()/mutableData<T>() with a dtype check, operator[].
//
// Extensions for the MI355X build: fp16/bf16 element types (core::Half / core::BFloat16 tags),
// a run-time dtype Reshape, and kDLROCM as a GPU device tag.
#pragma once

#include <cstdint>
#include <functional>
#include <memory>
#include <numeric>
#include <string>
#include <typeinfo>
#include <vector>

#include "core/dlpack.h"
#include "core/enforce.h"

namespace turbo_transformers {
namespace core {

struct Half { uint16_t x; };      // IEEE binary16 storage tag
struct BFloat16 { uint16_t x; };  // bfloat16 storage tag

template <typename T> struct DataTypeTrait;
template <> struct DataTypeTrait<float> { static constexpr DLDataType v{kDLFloat, 32, 1}; };
template <> struct DataTypeTrait<Half> { static constexpr DLDataType v{kDLFloat, 16, 1}; };
template <> struct DataTypeTrait<BFloat16> { static constexpr DLDataType v{kDLBfloat, 16, 1}; };
template <> struct DataTypeTrait<int64_t> { static constexpr DLDataType v{kDLInt, 64, 1}; };
template <> struct DataTypeTrait<int32_t> { static constexpr DLDataType v{kDLInt, 32, 1}; };
template <> struct DataTypeTrait<int8_t> { static constexpr DLDataType v{kDLInt, 8, 1}; };

inline bool SameDataType(DLDataType a, DLDataType b) { return a.code == b.code && a.bits == b.bits && a.lanes == b.lanes; }

// ttmi_dtype of a DLPack dtype, or -1.
int ToDeviceDType(DLDataType t);

// A new owning tensor whose buffer comes from allocator::Allocator (reference:
// NewDLPackTensor, core/tensor.cpp:55-94).
DLManagedTensor* NewDLPackTensor(const std::vector<int64_t>& shape, DLDataType dtype, DLDeviceType device,
                                 int device_id, const std::string& name = "");

template <typename T>
DLManagedTensor* NewDLPackTensorT(const std::vector<int64_t>& shape, DLDeviceType device = kDLCPU, int device_id = 0,
                                  const std::string& name = "") {
  return NewDLPackTensor(shape, DataTypeTrait<T>::v, device, device_id, name);
}

class Tensor {
 public:
  explicit Tensor(DLManagedTensor* tensor) : managed_(tensor) {}
  Tensor() : managed_(nullptr) {}
  ~Tensor() { Release(); }

  Tensor(Tensor&& o) noexcept { MoveFrom(o); }
  Tensor& operator=(Tensor&& o) {
    if (this == &o) TT_THROW("Tensor can not be assigned to itself!");
    Release();
    MoveFrom(o);
    return *this;
  }
  Tensor(const Tensor&) = delete;
  Tensor& operator=(const Tensor&) = delete;

  // Give up ownership (the consumer calls the deleter); the tensor becomes empty.
  DLManagedTensor* ToDLPack() {
    TT_ENFORCE(managed_ != nullptr, "Must own dltensor");
    DLManagedTensor* t = managed_;
    managed_ = nullptr;
    shadow_.reset();
    absmax_.reset();
    return t;
  }

  // Optional fp32 copy of the same values.  The bfloat16 layers attach it to their LayerNorm
  // outputs so that the next residual add reads unrounded values; it travels with the tensor
  // and is dropped whenever the buffer is handed out (ToDLPack) or re-shaped.
  const Tensor* shadow() const { return shadow_.get(); }
  Tensor* EnsureShadow();
  void DropShadow() { shadow_.reset(); }
  // Hand the fp32 copy to the caller (null when there is none); the tensor keeps its own buffer.
  std::unique_ptr<Tensor> TakeShadow() { return std::move(shadow_); }

  // Optional per-workgroup maxima of |value| (TTMI_ABSMAX_SLOTS floats on the device), attached by the kernel that
  // produced this tensor for the dynamic int8 quantisation of the Linear that consumes it (ttmi_*_absmax); like
  // the fp32 copy it travels with the tensor and is dropped whenever the buffer is handed out or re-shaped.
  const Tensor* absmax() const { return absmax_.get(); }
  Tensor* EnsureAbsmax();
  void DropAbsmax() { absmax_.reset(); }

  bool is_null() const { return managed_ == nullptr && !is_view_; }

  size_t n_dim() const { return (size_t)dl().ndim; }

  const int64_t& shape(int pos) const {
    const DLTensor& t = dl();
    if (pos < 0) pos = t.ndim + pos;
    TT_ENFORCE(pos >= 0 && pos < t.ndim, "The index(%d) is out of the range[0...%d]", pos, t.ndim - 1);
    return t.shape[pos];
  }

  int64_t numel() const {
    const DLTensor& t = dl();
    return std::accumulate(t.shape, t.shape + t.ndim, (int64_t)1, std::multiplies<int64_t>());
  }

  DLDeviceType device_type() const { return dl().device.device_type; }
  int device_id() const { return dl().device.device_id; }
  DLDevice device_ctx() const { return dl().device; }
  DLDataType dtype() const { return dl().dtype; }
  bool is_gpu() const { return IsGpu(device_type()); }
  size_t element_size() const { return (size_t)dl().dtype.bits / 8; }

  // Typed Reshape, as in the reference: (re)allocate when the held buffer is too small,
  // otherwise only rewrite the shape.
  template <typename T>
  T* Reshape(const std::vector<int64_t>& shape_list, DLDeviceType device_type, int device_id,
             const std::string& name = "Reshape") {
    ReshapeAs(DataTypeTrait<T>::v, shape_list, device_type, device_id, name);
    return mutableData<T>();
  }
  // Same with a run-time element type (activations follow the dtype of the weights).
  void* ReshapeAs(DLDataType dtype, const std::vector<int64_t>& shape_list, DLDeviceType device_type, int device_id,
                  const std::string& name = "Reshape");

  template <typename T>
  const T* data() const {
    const DLTensor& t = dl();
    TT_ENFORCE_EQ(t.byte_offset, (uint64_t)0, "byte_offset must be zero");
    TT_ENFORCE(SameDataType(t.dtype, DataTypeTrait<T>::v), "data type mismatch, request %s, actual (%d,%d)",
               typeid(T).name(), (int)t.dtype.code, (int)t.dtype.bits);
    return reinterpret_cast<const T*>(t.data);
  }
  template <typename T>
  // (asking for a writable pointer drops the attached maxima: whoever writes the buffer invalidates them, and a
  // producer that supplies new ones calls EnsureAbsmax() afterwards)
  T* mutableData() {
    absmax_.reset();
    return const_cast<T*>(data<T>());
  }

  const void* raw() const { return dl().data; }
  void* mutable_raw() {
    absmax_.reset();
    return dl().data;
  }

  // View of the n-th slice along dimension 0 (does not own memory).
  Tensor operator[](int64_t n);
  const Tensor operator[](int64_t n) const { return const_cast<Tensor*>(this)->operator[](n); }

 private:
  const DLTensor& dl() const {
    if (managed_) return managed_->dl_tensor;
    TT_ENFORCE(is_view_, "Tensor is null");
    return view_;
  }
  void Release() {
    if (managed_ && managed_->deleter) managed_->deleter(managed_);
    managed_ = nullptr;
    is_view_ = false;
    shadow_.reset();
    absmax_.reset();
  }
  void MoveFrom(Tensor& o) {
    shadow_ = std::move(o.shadow_);
    absmax_ = std::move(o.absmax_);
    managed_ = o.managed_;
    is_view_ = o.is_view_;
    view_ = o.view_;
    view_shape_ = std::move(o.view_shape_);
    if (is_view_) view_.shape = view_shape_.data();
    o.managed_ = nullptr;
    o.is_view_ = false;
  }

  DLManagedTensor* managed_ = nullptr;
  bool is_view_ = false;
  DLTensor view_{};
  std::vector<int64_t> view_shape_;
  std::unique_ptr<Tensor> shadow_;
  std::unique_ptr<Tensor> absmax_;
};

// Copy `numel` elements between buffers on the stream; host<->device copies synchronise
// (core/memory.cpp:34-81, core/tensor_copy.h).
void CopyBytes(void* dst, DLDeviceType dst_dev, const void* src, DLDeviceType src_dev, size_t bytes);

}  // namespace core
}  // namespace turbo_transformers
