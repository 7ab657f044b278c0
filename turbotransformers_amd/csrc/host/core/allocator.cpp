#include "core/allocator.h"

#include <cstdlib>

#include "core/enforce.h"
#include "ttmi.h"

namespace turbo_transformers {
namespace core {
namespace allocator {

Allocator& Allocator::GetInstance() {
  static Allocator a;
  return a;
}

size_t Allocator::RoundSize(size_t size) {
  if (size == 0) size = 1;
  constexpr size_t kSmall = 512, kLarge = 2u << 20, kThreshold = 1u << 20;
  const size_t q = size < kThreshold ? kSmall : kLarge;
  return (size + q - 1) / q * q;
}

void* Allocator::DeviceMalloc(size_t bytes) {
  if (device_limit_ != 0 && device_bytes_ + bytes > device_limit_) return nullptr;
  void* p = nullptr;
  if (ttmi_malloc(&p, bytes) != 0) return nullptr;
  device_bytes_ += bytes;
  ++stats_.device_mallocs;
  return p;
}

void* Allocator::allocate(size_t size, DLDeviceType dev, const std::string& name) {
  if (dev == kDLCPU) {
    void* p = nullptr;
    if (posix_memalign(&p, 64, size == 0 ? 64 : size) != 0) throw BadAlloc("posix_memalign failed for " + name);
    return p;
  }
  TT_ENFORCE(IsGpu(dev), "allocate: unsupported device type %d", (int)dev);
  const size_t rounded = RoundSize(size);
  std::lock_guard<std::mutex> g(mutex_);
  auto it = free_blocks_.lower_bound(rounded);
  if (it != free_blocks_.end() && it->first <= rounded + rounded / 4) {
    void* p = it->second;
    const size_t sz = it->first;
    free_blocks_.erase(it);
    live_blocks_[p] = sz;
    stats_.bytes_cached -= sz;
    stats_.bytes_live += sz;
    ++stats_.cache_hits;
    return p;
  }
  void* p = DeviceMalloc(rounded);
  if (p == nullptr) {
    // out of memory: drop the cache and try once more (naive_allocator.h:50-63)
    ++stats_.oom_retries;
    for (auto& kv : free_blocks_) {
      ttmi_free(kv.second);
      device_bytes_ -= kv.first;
    }
    free_blocks_.clear();
    stats_.bytes_cached = 0;
    p = DeviceMalloc(rounded);
    if (p == nullptr) throw BadAlloc("device out of memory allocating " + std::to_string(rounded) + " bytes for " + name);
  }
  live_blocks_[p] = rounded;
  stats_.bytes_live += rounded;
  return p;
}

void Allocator::free(void* mem, DLDeviceType dev, const std::string&) {
  if (mem == nullptr) return;
  if (dev == kDLCPU) {
    std::free(mem);
    return;
  }
  std::lock_guard<std::mutex> g(mutex_);
  auto it = live_blocks_.find(mem);
  TT_ENFORCE(it != live_blocks_.end(), "free of a pointer this allocator does not own");
  const size_t sz = it->second;
  live_blocks_.erase(it);
  free_blocks_.emplace(sz, mem);
  stats_.bytes_live -= sz;
  stats_.bytes_cached += sz;
}

void Allocator::FreeAllCached() {
  std::lock_guard<std::mutex> g(mutex_);
  if (free_blocks_.empty()) return;
  ttmi_stream_sync(nullptr);
  for (auto& kv : free_blocks_) {
    ttmi_free(kv.second);
    device_bytes_ -= kv.first;
  }
  free_blocks_.clear();
  stats_.bytes_cached = 0;
}

AllocatorStats Allocator::stats() {
  std::lock_guard<std::mutex> g(mutex_);
  return stats_;
}

void Allocator::set_schema(const std::string& schema) {
  // allocator_api.cpp:28-36 accepts "naive" and "model-aware"; the offline chunk planner of
  // the latter is not part of this build, so only "naive" is accepted.
  if (schema == "naive") {
    schema_ = schema;
    return;
  }
  if (schema == "model-aware") TT_THROW("allocator schema 'model-aware' is not built; use 'naive'");
  TT_THROW("no schema called %s", schema.c_str());
}

void reset_allocator_schema(const std::string& name) { Allocator::GetInstance().set_schema(name); }

void bert_opt_mem_allocate_api(int64_t, int64_t, int64_t, int64_t, int64_t, const std::string&) {
  // Only meaningful for the model-aware schema (allocator_api.cpp:112-125): a no-op under "naive".
  TT_ENFORCE(Allocator::GetInstance().schema() == "naive", "unexpected allocator schema");
}

}  // namespace allocator
}  // namespace core
}  // namespace turbo_transformers
