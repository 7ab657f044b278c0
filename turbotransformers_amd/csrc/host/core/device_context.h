// Process-wide device state: the stream every kernel is enqueued on, and small per-batch
// device tables for variable-length (smart) batches.  Stands in for core::CUDADeviceContext
// (turbo_transformers/core/cuda_device_context.cpp:23-46); no BLAS handle is needed because
// the GEMMs are hand-written kernels.
//
// The stream defaults to the legacy default stream, which is also torch's default current
// stream; Python passes torch's current stream before each forward (set_stream), so work
// queued by torch on the inputs is ordered before the kernels here.
#pragma once

#include <cstdint>
#include <mutex>
#include <vector>

namespace turbo_transformers {
namespace core {

class DeviceContext {
 public:
  static DeviceContext& GetInstance();

  void* stream() const { return stream_; }
  // Switching to another stream first drains the old one: cached state (packed weights, recycled allocator blocks,
  // the batch tables below) was produced by work on the old stream and carries no other dependency.
  void set_stream(void* s);
  void Wait() const;  // synchronise the stream and surface asynchronous kernel errors

  int compute_units();

  // Device-side description of a packed batch: cu_seqlens[B+1] and, for each packed token,
  // its row in the zero-padded [B, max_seq] layout.  Cached on the list of lengths, so the
  // twelve layers of one forward upload it once.
  struct SeqPlan {
    const int32_t* cu_seqlens = nullptr;
    const int32_t* token_rows = nullptr;
    int64_t batch = 0, max_seq = 0, total = 0;
  };
  SeqPlan GetSeqPlan(const std::vector<int64_t>& lens);

 private:
  DeviceContext() = default;
  void* stream_ = nullptr;
  int compute_units_ = -1;
  std::mutex plan_mutex_;
  std::vector<int64_t> plan_lens_;
  int32_t* plan_cu_ = nullptr;
  int32_t* plan_rows_ = nullptr;
  // Pinned staging words of the cu_seqlens upload: a small ring, each slot with the event recorded behind its copy, so
  // that a new list of lengths waits only for the copy that used its slot four uploads ago, never for the stream.
  static constexpr int kPlanSlots = 4;
  struct StagingSlot {
    int32_t* words = nullptr;
    void* copied = nullptr;  // event
    bool in_use = false;
  };
  StagingSlot plan_slots_[kPlanSlots];
  int plan_next_slot_ = 0;
  int64_t plan_cu_cap_ = 0, plan_rows_cap_ = 0;
  void* plan_stream_ = nullptr;
};

}  // namespace core
}  // namespace turbo_transformers
