#include "core/device_context.h"

#include <algorithm>
#include <numeric>

#include "core/enforce.h"
#include "ttmi.h"

namespace turbo_transformers {
namespace core {

DeviceContext& DeviceContext::GetInstance() {
  static DeviceContext ctx;
  return ctx;
}

void DeviceContext::set_stream(void* s) {
  if (s == stream_) return;
  TT_DEVICE_CALL(ttmi_stream_sync(stream_));
  stream_ = s;
}

void DeviceContext::Wait() const {
  TT_DEVICE_CALL(ttmi_stream_sync(stream_));
  TT_DEVICE_CALL(ttmi_check_async());
}

int DeviceContext::compute_units() {
  if (compute_units_ < 0) {
    int cu = 0;
    TT_DEVICE_CALL(ttmi_device_info(nullptr, 0, &cu, nullptr, nullptr, nullptr));
    compute_units_ = cu;
  }
  return compute_units_;
}

DeviceContext::SeqPlan DeviceContext::GetSeqPlan(const std::vector<int64_t>& lens) {
  std::lock_guard<std::mutex> g(plan_mutex_);
  TT_ENFORCE(!lens.empty(), "seq_len_list must not be empty");
  const int64_t batch = (int64_t)lens.size();
  const int64_t total = std::accumulate(lens.begin(), lens.end(), (int64_t)0);
  const int64_t max_seq = *std::max_element(lens.begin(), lens.end());
  if (!(lens == plan_lens_ && plan_stream_ == stream_)) {
    // The device tables are rewritten in stream order, behind the kernels that still read the previous batch's.
    if (batch + 1 > plan_cu_cap_) {
      // Retired buffers may still be read by kernels in flight: drain the stream first (growth is rare).
      TT_DEVICE_CALL(ttmi_stream_sync(stream_));
      if (plan_cu_) TT_DEVICE_CALL(ttmi_free(plan_cu_));
      plan_cu_cap_ = std::max<int64_t>(64, 2 * (batch + 1));
      TT_DEVICE_CALL(ttmi_malloc(reinterpret_cast<void**>(&plan_cu_), plan_cu_cap_ * sizeof(int32_t)));
      for (StagingSlot& slot : plan_slots_) {
        if (slot.words) TT_DEVICE_CALL(ttmi_host_free(slot.words));
        TT_DEVICE_CALL(ttmi_host_malloc(reinterpret_cast<void**>(&slot.words), plan_cu_cap_ * sizeof(int32_t)));
        if (slot.copied == nullptr) TT_DEVICE_CALL(ttmi_event_create(&slot.copied));
        slot.in_use = false;
      }
    }
    if (total > plan_rows_cap_) {
      TT_DEVICE_CALL(ttmi_stream_sync(stream_));
      if (plan_rows_) TT_DEVICE_CALL(ttmi_free(plan_rows_));
      plan_rows_cap_ = std::max<int64_t>(4096, 2 * total);
      TT_DEVICE_CALL(ttmi_malloc(reinterpret_cast<void**>(&plan_rows_), plan_rows_cap_ * sizeof(int32_t)));
    }
    StagingSlot& slot = plan_slots_[plan_next_slot_];
    plan_next_slot_ = (plan_next_slot_ + 1) % kPlanSlots;
    // the pinned words are read by an asynchronous copy: the one that used this slot last must be done
    if (slot.in_use) TT_DEVICE_CALL(ttmi_event_sync(slot.copied));
    TT_DEVICE_CALL(ttmi_build_cu_seqlens(lens.data(), batch, slot.words, plan_cu_, stream_));
    TT_DEVICE_CALL(ttmi_event_record(slot.copied, stream_));
    slot.in_use = true;
    if (total > 0) TT_DEVICE_CALL(ttmi_build_token_rows(plan_cu_, batch, max_seq, total, plan_rows_, stream_));
    plan_lens_ = lens;
    plan_stream_ = stream_;
  }
  SeqPlan p;
  p.cu_seqlens = plan_cu_;
  p.token_rows = plan_rows_;
  p.batch = batch;
  p.max_seq = max_seq;
  p.total = total;
  return p;
}

}  // namespace core
}  // namespace turbo_transformers
