// Minimal DLPack ABI (the unversioned DLManagedTensor exchange that torch.utils.dlpack
// speaks), declared here so the host layer needs neither the dlpack submodule nor torch
// headers.  The reference was written against the pre-0.6 names (DLContext / kDLGPU,
// core/tensor.h:197,204); torch on ROCm tags device memory kDLROCM, so both map to "GPU".
#pragma once

#include <cstdint>

extern "C" {

typedef enum {
  kDLCPU = 1,
  kDLCUDA = 2,
  kDLGPU = 2,  // legacy name used throughout the reference
  kDLCUDAHost = 3,
  kDLROCM = 10,
  kDLROCMHost = 11,
} DLDeviceType;

typedef struct {
  DLDeviceType device_type;
  int32_t device_id;
} DLDevice;

typedef enum {
  kDLInt = 0U,
  kDLUInt = 1U,
  kDLFloat = 2U,
  kDLOpaqueHandle = 3U,
  kDLBfloat = 4U,
  kDLComplex = 5U,
  kDLBool = 6U,
} DLDataTypeCode;

typedef struct {
  uint8_t code;
  uint8_t bits;
  uint16_t lanes;
} DLDataType;

typedef struct {
  void* data;
  DLDevice device;
  int32_t ndim;
  DLDataType dtype;
  int64_t* shape;
  int64_t* strides;
  uint64_t byte_offset;
} DLTensor;

typedef struct DLManagedTensor {
  DLTensor dl_tensor;
  void* manager_ctx;
  void (*deleter)(struct DLManagedTensor* self);
} DLManagedTensor;

}  // extern "C"

namespace turbo_transformers {
namespace core {
inline bool IsGpu(DLDeviceType t) { return t == kDLCUDA || t == kDLROCM; }
}  // namespace core
}  // namespace turbo_transformers
