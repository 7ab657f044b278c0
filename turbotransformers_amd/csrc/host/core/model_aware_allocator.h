// Model-aware activation placement: all activation buffers of a BERT forward are given fixed
// offsets inside a few large device chunks, computed from the tensors' sizes and lifetimes
// before the forward runs, so the steady state allocates nothing and every encoder layer
// reuses the same addresses.  Counterpart of the reference's model-aware schema
// (turbo_transformers/core/allocator/model_aware_allocator.h:34-117,
//  model_aware_memory_scheduler.{h,cpp}, bert_config.cpp:41-93).
//
// The planner is a plain function over value types so that it can be tested without a device.
#pragma once

#include <cstdint>
#include <functional>
#include <map>
#include <set>
#include <string>
#include <vector>

namespace turbo_transformers {
namespace core {
namespace allocator {

constexpr int64_t kDefaultChunkSize = 2 * 1024 * 1024;  // model_aware_memory_scheduler.h:30
constexpr double kChunkScale = 1.2;                     // model_aware_memory_scheduler.h:31
constexpr int64_t kPlacementAlign = 256;                // every offset keeps 16-byte vector access legal

// A tensor is live during operators [start_op, end_op] (inclusive) and needs `size` bytes.
struct TensorRecord {
  std::string name;
  int64_t start_op = 0;
  int64_t end_op = 0;
  int64_t size = 0;
};

struct Placement {
  int chunk = -1;  // index into the chunk-size list
  int64_t offset = 0;
};

// Greedy-by-size placement into chunks (model_aware_memory_scheduler.cpp:34-120).
// `records` are taken in the given order (callers sort by size, largest first).  Each record goes
// into the first chunk, smallest chunk first, that has room among the records already placed there
// whose lifetimes intersect its own: the tightest gap between two such neighbours that fits, else
// the space behind the last of them.  When no chunk fits, a chunk of
// max(kDefaultChunkSize, 1.2 * size rounded up to 32) bytes is appended.
// `chunk_sizes` may already hold chunks from an earlier plan (they are reused, emptied first);
// on return `chunk_used[i]` says whether chunk i received any tensor.
void ChunkedGreedyBySizeOffsetCalculation(const std::vector<TensorRecord>& records, std::vector<int64_t>* chunk_sizes,
                                          std::vector<Placement>* placements, std::vector<bool>* chunk_used);

// True when no two records that are live at the same time overlap in memory, every record lies
// inside its chunk and every offset is aligned (the predicate of bert_allocator_test.cpp:30-66).
bool PlacementIsValid(const std::vector<TensorRecord>& records, const std::vector<int64_t>& chunk_sizes,
                      const std::vector<Placement>& placements);

// Usage records of the activations of this build's BERT forward (names are the `name` arguments
// the layers pass to Tensor::Reshape), sorted by size, largest first.  Sizes are for 4-byte
// elements, which also covers fp16/bf16.  All encoder layers share one set of records.
std::vector<TensorRecord> BertTensorUsageRecords(int64_t batch_size, int64_t seq_len, int64_t num_head,
                                                 int64_t hidden_size, int64_t num_layer);

// Keeps the current plan and the device chunks behind it.
class ModelAwarePlan {
 public:
  using AllocFn = std::function<void*(size_t)>;
  using FreeFn = std::function<void(void*)>;
  ModelAwarePlan(AllocFn alloc, FreeFn free) : alloc_(std::move(alloc)), free_(std::move(free)) {}
  ~ModelAwarePlan();

  // Re-plan for a new input shape; chunks that are still large enough are kept, unused ones freed.
  void Reset(int64_t batch_size, int64_t seq_len, int64_t num_head, int64_t hidden_size, int64_t num_layer);
  bool Has(const std::string& name) const { return position_.count(name) != 0; }
  // Address of a planned tensor; throws when `size` exceeds what was planned for it.
  void* Address(const std::string& name, size_t size) const;

  size_t chunk_count() const { return chunk_mem_.size(); }
  int64_t chunk_bytes() const;

 private:
  struct Position {
    int chunk;
    int64_t offset;
    int64_t size;
  };
  AllocFn alloc_;
  FreeFn free_;
  std::vector<int64_t> chunk_sizes_;
  std::vector<void*> chunk_mem_;
  std::map<std::string, Position> position_;
};

}  // namespace allocator
}  // namespace core
}  // namespace turbo_transformers
