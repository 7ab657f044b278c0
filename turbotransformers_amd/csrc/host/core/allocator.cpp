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

// Chunks of the model-aware plan come straight from the device (they are few, large and long-lived)
// and are returned only after the device has drained, since kernels may still be using them.
Allocator::Allocator()
    : plan_(new ModelAwarePlan(
          [](size_t bytes) -> void* {
            void* p = nullptr;
            return ttmi_malloc(&p, bytes) == 0 ? p : nullptr;
          },
          [](void* p) {
            ttmi_stream_sync(nullptr);
            ttmi_free(p);
          })) {}

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
  if (IsGpu(dev) && is_activation(name)) {
    std::lock_guard<std::mutex> g(mutex_);
    return plan_->Address(name, size);
  }
  return NaiveAllocate(size, dev, name);
}

void* Allocator::NaiveAllocate(size_t size, DLDeviceType dev, const std::string& name) {
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
  TT_ENFORCE(it != live_blocks_.end(), "free of a pointer this allocator does not own (planned activations are never freed)");
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
  // allocator_api.cpp:64-81: "naive" and "model-aware" are the registered schemas
  TT_ENFORCE(schema == "naive" || schema == "model-aware", "no schema called %s", schema.c_str());
  std::lock_guard<std::mutex> g(mutex_);
  schema_ = schema;
}

bool Allocator::is_activation(const std::string& name) {
  std::lock_guard<std::mutex> g(mutex_);
  return schema_ == "model-aware" && plan_->Has(name);
}

void Allocator::set_config(int64_t batch_size, int64_t seq_len, int64_t num_head, int64_t hidden_size, int64_t num_layer) {
  std::lock_guard<std::mutex> g(mutex_);
  plan_->Reset(batch_size, seq_len, num_head, hidden_size, num_layer);
}

std::pair<size_t, int64_t> Allocator::model_aware_chunks() {
  std::lock_guard<std::mutex> g(mutex_);
  return {plan_->chunk_count(), plan_->chunk_bytes()};
}

void reset_allocator_schema(const std::string& name) { Allocator::GetInstance().set_schema(name); }

void bert_opt_mem_allocate_api(int64_t batch_size, int64_t seq_len, int64_t num_head, int64_t hidden_size, int64_t num_layer,
                               const std::string& dev_str) {
  // allocator_api.cpp:112-118.  Only device activations are planned here; host tensors of this
  // build are a few ids and always come from the heap.
  TT_ENFORCE(dev_str == "GPU" || dev_str == "CPU", "device must be \"GPU\" or \"CPU\"");
  if (dev_str == "GPU") Allocator::GetInstance().set_config(batch_size, seq_len, num_head, hidden_size, num_layer);
}

}  // namespace allocator
}  // namespace core
}  // namespace turbo_transformers
