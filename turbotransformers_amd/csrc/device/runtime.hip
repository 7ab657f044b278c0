// Runtime part of the C ABI: device bring-up, raw memory, copies, streams, events and the
// error plumbing shared by every kernel file.
#include "common.h"

#include <atomic>
#include <cstdlib>
#include <cstring>

namespace ttmi {

namespace {
const char* const kSwitchNames[kNumKernelSwitches] = {"TTMI_LARGE_TILE", "TTMI_WAVE_KERNEL", "TTMI_ATTENTION_WAVES",
                                                       "TTMI_STATIC_SCRATCH_LIMIT", "TTMI_W4_A_STAGES", "TTMI_W4_SPLITK"};
struct KernelSwitches {
  std::atomic<int> value[kNumKernelSwitches];
  KernelSwitches() {
    for (int i = 0; i < kNumKernelSwitches; ++i) {
      const char* text = std::getenv(kSwitchNames[i]);
      value[i].store(text != nullptr && text[0] != 0 ? std::atoi(text) : kSwitchUnset, std::memory_order_relaxed);
    }
  }
};
KernelSwitches& kernel_switches() {
  static KernelSwitches s;  // the environment is read here, once
  return s;
}
}  // namespace

int kernel_switch(KernelSwitch which) { return kernel_switches().value[which].load(std::memory_order_relaxed); }

static thread_local std::string g_last_error;

void set_error(const std::string& msg) { g_last_error = msg; }

int fail(int code, const std::string& msg) {
  g_last_error = msg;
  return code;
}

int check_hip(hipError_t e, const char* what) {
  if (e == hipSuccess) return 0;
  g_last_error = std::string(what) + ": " + hipGetErrorString(e);
  return e == hipErrorOutOfMemory ? TTMI_ENOMEM : TTMI_EDEVICE;
}

// One pinned, device-mapped int per process.  Kernels raise it with an ordinary vector
// store; the host reads it after a stream sync.
int* async_error_flag() {
  static int* flag = [] {
    int* p = nullptr;
    if (hipHostMalloc(reinterpret_cast<void**>(&p), sizeof(int), hipHostMallocMapped) != hipSuccess) return (int*)nullptr;
    *p = 0;
    return p;
  }();
  return flag;
}

template <typename T>
__global__ void fill_kernel(T* data, int64_t n, T value) {
  int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (; i < n; i += stride) data[i] = value;
}

}  // namespace ttmi

using namespace ttmi;

extern "C" {

const char* ttmi_last_error(void) { return g_last_error.c_str(); }

int ttmi_set_kernel_switch(const char* name, int value) {
  TTMI_REQUIRE(name != nullptr, "switch name is null");
  for (int i = 0; i < kNumKernelSwitches; ++i) {
    if (std::strcmp(name, kSwitchNames[i]) == 0) {
      kernel_switches().value[i].store(value, std::memory_order_relaxed);
      return 0;
    }
  }
  return fail(TTMI_EINVAL, std::string("unknown kernel switch ") + name);
}

int ttmi_device_count(int* count) {
  TTMI_REQUIRE(count != nullptr, "count is null");
  hipError_t e = hipGetDeviceCount(count);
  if (e != hipSuccess) {
    *count = 0;
    (void)hipGetLastError();
  }
  return 0;
}

int ttmi_set_device(int device) {
  TTMI_HIP(hipSetDevice(device));
  return 0;
}

int ttmi_device_info(char* name, int name_len, int* compute_units, int* clock_khz, int64_t* hbm_bytes,
                     int* lds_bytes_per_cu) {
  int dev = 0;
  TTMI_HIP(hipGetDevice(&dev));
  hipDeviceProp_t prop;
  TTMI_HIP(hipGetDeviceProperties(&prop, dev));
  if (name && name_len > 0) {
    std::string full = std::string(prop.name) + " (" + prop.gcnArchName + ")";
    std::strncpy(name, full.c_str(), name_len - 1);
    name[name_len - 1] = 0;
  }
  if (compute_units) *compute_units = prop.multiProcessorCount;
  if (clock_khz) *clock_khz = prop.clockRate;
  if (hbm_bytes) *hbm_bytes = (int64_t)prop.totalGlobalMem;
  if (lds_bytes_per_cu) *lds_bytes_per_cu = (int)prop.maxSharedMemoryPerMultiProcessor;
  return 0;
}

int ttmi_mem_info(int64_t* free_bytes, int64_t* total_bytes) {
  size_t f = 0, t = 0;
  TTMI_HIP(hipMemGetInfo(&f, &t));
  if (free_bytes) *free_bytes = (int64_t)f;
  if (total_bytes) *total_bytes = (int64_t)t;
  return 0;
}

int ttmi_malloc(void** ptr, size_t bytes) {
  TTMI_REQUIRE(ptr != nullptr, "ptr is null");
  *ptr = nullptr;
  if (bytes == 0) return 0;
  hipError_t e = hipMalloc(ptr, bytes);
  if (e != hipSuccess) {
    (void)hipGetLastError();  // clear the sticky error so the caller may free cache and retry
    *ptr = nullptr;
    return check_hip(e, "hipMalloc");
  }
  return 0;
}

int ttmi_free(void* ptr) {
  if (ptr) TTMI_HIP(hipFree(ptr));
  return 0;
}

int ttmi_host_malloc(void** ptr, size_t bytes) {
  TTMI_REQUIRE(ptr != nullptr, "ptr is null");
  TTMI_HIP(hipHostMalloc(ptr, bytes, hipHostMallocDefault));
  return 0;
}

int ttmi_host_free(void* ptr) {
  if (ptr) TTMI_HIP(hipHostFree(ptr));
  return 0;
}

static hipMemcpyKind to_kind(int kind) {
  switch (kind) {
    case TTMI_H2D: return hipMemcpyHostToDevice;
    case TTMI_D2H: return hipMemcpyDeviceToHost;
    default: return hipMemcpyDeviceToDevice;
  }
}

int ttmi_memcpy_async(void* dst, const void* src, size_t bytes, int kind, void* stream) {
  if (bytes == 0) return 0;
  TTMI_HIP(hipMemcpyAsync(dst, src, bytes, to_kind(kind), (hipStream_t)stream));
  return 0;
}

int ttmi_memcpy(void* dst, const void* src, size_t bytes, int kind, void* stream) {
  if (bytes == 0) return 0;
  TTMI_HIP(hipMemcpyAsync(dst, src, bytes, to_kind(kind), (hipStream_t)stream));
  TTMI_HIP(hipStreamSynchronize((hipStream_t)stream));
  return 0;
}

int ttmi_memset_zero(void* dst, size_t bytes, void* stream) {
  if (bytes == 0) return 0;
  TTMI_REQUIRE((reinterpret_cast<uintptr_t>(dst) & 3) == 0 && (bytes & 3) == 0,
               "memset_zero needs 4-byte aligned pointer and size");
  const int64_t n = (int64_t)(bytes / 4);
  const int block = 256;
  const int grid = (int)std::min<int64_t>(ceil_div(n, block), 4096);
  hipLaunchKernelGGL(fill_kernel<uint32_t>, dim3(grid), dim3(block), 0, (hipStream_t)stream,
                     (uint32_t*)dst, n, 0u);
  return launch_status("memset_zero");
}

int ttmi_stream_create(void** stream) {
  TTMI_REQUIRE(stream != nullptr, "stream is null");
  hipStream_t s;
  TTMI_HIP(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));
  *stream = (void*)s;
  return 0;
}
int ttmi_stream_destroy(void* stream) {
  if (stream) TTMI_HIP(hipStreamDestroy((hipStream_t)stream));
  return 0;
}
int ttmi_stream_sync(void* stream) {
  TTMI_HIP(hipStreamSynchronize((hipStream_t)stream));
  return 0;
}
int ttmi_event_create(void** event) {
  TTMI_REQUIRE(event != nullptr, "event is null");
  hipEvent_t e;
  TTMI_HIP(hipEventCreate(&e));
  *event = (void*)e;
  return 0;
}
int ttmi_event_destroy(void* event) {
  if (event) TTMI_HIP(hipEventDestroy((hipEvent_t)event));
  return 0;
}
int ttmi_event_record(void* event, void* stream) {
  TTMI_HIP(hipEventRecord((hipEvent_t)event, (hipStream_t)stream));
  return 0;
}
int ttmi_event_sync(void* event) {
  TTMI_HIP(hipEventSynchronize((hipEvent_t)event));
  return 0;
}
int ttmi_event_elapsed_ms(void* start, void* stop, float* ms) {
  TTMI_HIP(hipEventElapsedTime(ms, (hipEvent_t)start, (hipEvent_t)stop));
  return 0;
}

int ttmi_check_async(void) {
  int* flag = async_error_flag();
  if (flag && *flag != 0) {
    *flag = 0;
    return fail(TTMI_EINDEX, "embedding id out of range");
  }
  return 0;
}

int ttmi_fill_i64(int64_t* data, int64_t n, int64_t value, void* stream) {
  if (n <= 0) return 0;
  const int grid = (int)std::min<int64_t>(ceil_div(n, 256), 4096);
  hipLaunchKernelGGL(fill_kernel<int64_t>, dim3(grid), dim3(256), 0, (hipStream_t)stream, data, n, value);
  return launch_status("fill_i64");
}

int ttmi_fill_f32(float* data, int64_t n, float value, void* stream) {
  if (n <= 0) return 0;
  const int grid = (int)std::min<int64_t>(ceil_div(n, 256), 4096);
  hipLaunchKernelGGL(fill_kernel<float>, dim3(grid), dim3(256), 0, (hipStream_t)stream, data, n, value);
  return launch_status("fill_f32");
}

}  // extern "C"
