// Process-wide activation allocator.  Same interface as the reference's allocator::Allocator
// (turbo_transformers/core/allocator/allocator_api.h:34-66): allocate(size, dev, name) /
// free(ptr, dev, name), schema selected by name.
//
//   "naive"  CPU: posix_memalign(64) (core/memory.cpp:24-31).
//            GPU: a caching allocator on hipMalloc (through the C ABI) in place of
//            cub::CachingDeviceAllocator (allocator/naive_allocator.h:36-100).  Blocks are
//            rounded to 512 B (< 1 MiB) or 2 MiB multiples and cached on free; a request
//            takes the smallest cached block that fits with at most 25 % slack.  When
//            hipMalloc fails, every cached block is released and the request retried once
//            (naive_allocator.h:50-63).  Reuse is ordered by the single work stream.
//
//   "model-aware"  device tensors whose name is one of the planned BERT activations live at a fixed
//            offset of a few large chunks (core/model_aware_allocator.h), decided by
//            bert_opt_mem_allocate_api(batch, seq, heads, hidden, layers, dev) before the forward;
//            they are never freed individually.  Everything else goes the "naive" way.
//
// With 288 GB of HBM per GPU the cache is never trimmed on its own; FreeAllCached() does it.
#pragma once

#include <cstddef>
#include <map>
#include <memory>
#include <mutex>
#include <string>
#include <unordered_map>

#include "core/dlpack.h"
#include "core/model_aware_allocator.h"

namespace turbo_transformers {
namespace core {
namespace allocator {

class BadAlloc : public std::exception {
 public:
  explicit BadAlloc(std::string msg) : msg_(std::move(msg)) {}
  const char* what() const noexcept override { return msg_.c_str(); }

 private:
  std::string msg_;
};

struct AllocatorStats {
  size_t device_mallocs = 0;     // calls that reached hipMalloc
  size_t cache_hits = 0;         // requests served from the cache
  size_t bytes_live = 0;         // handed out
  size_t bytes_cached = 0;       // held in the free lists
  size_t oom_retries = 0;
};

class Allocator {
 public:
  static Allocator& GetInstance();

  void* allocate(size_t size, DLDeviceType dev, const std::string& name);
  void free(void* mem, DLDeviceType dev, const std::string& name);

  void set_schema(const std::string& schema);
  const std::string& schema() const { return schema_; }
  // True when the model-aware schema is active and `name` is one of its planned activations:
  // such memory is owned by the plan, not by the tensor that points at it.
  bool is_activation(const std::string& name);
  // Plan the activations of a BERT of this shape (allocator_api.cpp:83-88).
  void set_config(int64_t batch_size, int64_t seq_len, int64_t num_head, int64_t hidden_size, int64_t num_layer);
  // Chunks held by the model-aware plan (count, bytes).
  std::pair<size_t, int64_t> model_aware_chunks();

  void FreeAllCached();
  AllocatorStats stats();
  // Test hook: cap on bytes obtained from the device (0 = no cap) to exercise the OOM path.
  void set_device_limit_for_test(size_t bytes) { device_limit_ = bytes; }

  static size_t RoundSize(size_t size);

 private:
  Allocator();
  ~Allocator() { plan_.release(); }  // chunks are left to process teardown: the device runtime may already be gone
  void* DeviceMalloc(size_t bytes);
  void* NaiveAllocate(size_t size, DLDeviceType dev, const std::string& name);

  std::string schema_ = "naive";
  std::mutex mutex_;
  std::multimap<size_t, void*> free_blocks_;             // size -> ptr
  std::unordered_map<void*, size_t> live_blocks_;        // ptr -> rounded size
  AllocatorStats stats_;
  size_t device_limit_ = 0;
  size_t device_bytes_ = 0;
  std::unique_ptr<ModelAwarePlan> plan_;
};

// Free functions with the reference's names (allocator_api.cpp:112-125).
void reset_allocator_schema(const std::string& name);
void bert_opt_mem_allocate_api(int64_t batch_size, int64_t seq_len, int64_t num_head, int64_t hidden_size,
                               int64_t num_layer, const std::string& dev_str);

}  // namespace allocator
}  // namespace core
}  // namespace turbo_transformers
