#include "core/model_aware_allocator.h"

#include <algorithm>
#include <limits>
#include <numeric>

#include "core/enforce.h"

namespace turbo_transformers {
namespace core {
namespace allocator {

namespace {

struct Slot {  // a record already placed in a chunk
  int64_t offset, size, start_op, end_op;
};

int64_t AlignUp(int64_t v, int64_t a) { return (v + a - 1) / a * a; }

// Best offset for `t` inside one chunk, or -1.  `slots` is kept sorted by offset.
int64_t FitIntoChunk(const TensorRecord& t, int64_t t_size, int64_t chunk_size, const std::vector<Slot>& slots) {
  int64_t prev_end = 0, best = -1, smallest_gap = std::numeric_limits<int64_t>::max();
  for (const Slot& x : slots) {
    if (std::max(t.start_op, x.start_op) > std::min(t.end_op, x.end_op)) continue;  // never live together
    const int64_t gap = x.offset - prev_end;
    if (gap >= t_size && gap < smallest_gap) {
      smallest_gap = gap;
      best = prev_end;
    }
    prev_end = std::max(prev_end, x.offset + x.size);
  }
  if (best < 0 && chunk_size - prev_end >= t_size) best = prev_end;
  return best;
}

}  // namespace

void ChunkedGreedyBySizeOffsetCalculation(const std::vector<TensorRecord>& records, std::vector<int64_t>* chunk_sizes,
                                          std::vector<Placement>* placements, std::vector<bool>* chunk_used) {
  placements->assign(records.size(), Placement{});
  std::vector<std::vector<Slot>> slots(chunk_sizes->size());
  for (size_t r = 0; r < records.size(); ++r) {
    const TensorRecord& t = records[r];
    TT_ENFORCE(t.size >= 0 && t.start_op <= t.end_op, "bad usage record for %s", t.name.c_str());
    const int64_t t_size = AlignUp(std::max<int64_t>(t.size, 1), kPlacementAlign);
    // visit chunks from the smallest to the largest (stable in creation order)
    std::vector<int> order(chunk_sizes->size());
    std::iota(order.begin(), order.end(), 0);
    std::stable_sort(order.begin(), order.end(), [&](int a, int b) { return (*chunk_sizes)[a] < (*chunk_sizes)[b]; });
    int chosen = -1;
    int64_t offset = -1;
    for (int c : order) {
      offset = FitIntoChunk(t, t_size, (*chunk_sizes)[c], slots[c]);
      if (offset >= 0) {
        chosen = c;
        break;
      }
    }
    if (chosen < 0) {
      const int64_t scaled = (static_cast<int64_t>(t_size * kChunkScale) + 31) / 32 * 32;
      chunk_sizes->push_back(AlignUp(std::max(kDefaultChunkSize, scaled), kPlacementAlign));
      slots.emplace_back();
      chosen = (int)chunk_sizes->size() - 1;
      offset = 0;
    }
    Slot s{offset, t_size, t.start_op, t.end_op};
    auto& list = slots[chosen];
    list.insert(std::upper_bound(list.begin(), list.end(), s, [](const Slot& a, const Slot& b) { return a.offset < b.offset; }), s);
    (*placements)[r] = Placement{chosen, offset};
  }
  chunk_used->assign(chunk_sizes->size(), false);
  for (size_t c = 0; c < slots.size(); ++c) (*chunk_used)[c] = !slots[c].empty();
}

bool PlacementIsValid(const std::vector<TensorRecord>& records, const std::vector<int64_t>& chunk_sizes,
                      const std::vector<Placement>& placements) {
  if (placements.size() != records.size()) return false;
  for (size_t i = 0; i < records.size(); ++i) {
    const Placement& p = placements[i];
    if (p.chunk < 0 || p.chunk >= (int)chunk_sizes.size()) return false;
    if (p.offset < 0 || p.offset % kPlacementAlign != 0 || p.offset + records[i].size > chunk_sizes[p.chunk]) return false;
    for (size_t j = 0; j < i; ++j) {
      const Placement& q = placements[j];
      if (q.chunk != p.chunk) continue;
      const bool together = std::max(records[i].start_op, records[j].start_op) <= std::min(records[i].end_op, records[j].end_op);
      const bool overlap = std::max(p.offset, q.offset) < std::min(p.offset + records[i].size, q.offset + records[j].size);
      if (together && overlap) return false;
    }
  }
  return true;
}

std::vector<TensorRecord> BertTensorUsageRecords(int64_t batch_size, int64_t seq_len, int64_t num_head,
                                                 int64_t hidden_size, int64_t num_layer) {
  TT_ENFORCE(batch_size > 0 && seq_len > 0 && num_head > 0 && hidden_size > 0 && num_layer > 0, "bad model shape");
  const int64_t item = 4, id_bytes = 8;
  const int64_t tokens = batch_size * seq_len;
  const int64_t seq8 = (seq_len + 7) / 8 * 8;  // V may be kept transposed with the sequence padded to 8
  const int64_t hidden_bytes = tokens * hidden_size * item;
  const int64_t v_bytes = batch_size * seq8 * hidden_size * item;
  const int64_t score_bytes = batch_size * num_head * seq_len * seq_len * item;
  const int64_t ids_bytes = tokens * id_bytes;

  // Operator clock.  0: PrepareBertMasks, 1: embedding, then per layer (s = 2, the same for
  // every layer): s+0 QKV GEMM+split, s+1 QK^T or the fused attention core, s+2 softmax,
  // s+3 P.V (+ pad removal), s+4 output projection, s+5 AddBiasLayerNorm, s+6 FFN1,
  // s+7 FFN2, s+8 AddBiasLayerNorm; 11: pooler, 12: sequence pool.
  const int64_t s = 2, last = 12;
  std::vector<TensorRecord> r;
  auto add = [&](const char* name, int64_t a, int64_t b, int64_t bytes) { r.push_back(TensorRecord{name, a, b, bytes}); };
  add("PrepareBertMasks/possitionids/Reshape", 0, 1, ids_bytes);
  add("PrepareBertMasks/seqids/Reshape", 0, 1, ids_bytes);
  add("PrepareBertMasks/attmask/Reshape", 0, 0, ids_bytes);
  add("PrepareBertMasks/extendedattnmask/Reshape", 0, last, tokens * item);
  // hidden states: the embedding output and every layer's output share this buffer (bert_output.cpp:41-46)
  add("BERTEmbedding/Reshape", 1, last, hidden_bytes);
  add("self/q/Reshape", s + 0, s + 1, hidden_bytes);
  add("self/k/Reshape", s + 0, s + 1, hidden_bytes);
  add("self/v/Reshape", s + 0, s + 3, v_bytes);
  add("batch_gemm3/Reshape", s + 1, s + 3, score_bytes);         // scores / probabilities (unfused core only)
  add("ApplyMaskAndSoftmax/Reshape", s + 3, s + 4, hidden_bytes);  // padded context of a packed batch
  add("batch_gemm4/Reshape", s + 1, s + 4, hidden_bytes);         // merged context
  add("gemm5/Reshape", s + 4, s + 8, hidden_bytes);               // attention output, residual of the FFN
  add("BertIntermediate/Reshape", s + 6, s + 7, hidden_bytes * 4);
  add("BertPooler/Reshape", 11, last, batch_size * hidden_size * item);
  add("SeqPool/Reshape", 11, last, batch_size * hidden_size * item);
  std::stable_sort(r.begin(), r.end(), [](const TensorRecord& a, const TensorRecord& b) { return a.size > b.size; });
  return r;
}

ModelAwarePlan::~ModelAwarePlan() {
  for (void* p : chunk_mem_)
    if (p != nullptr) free_(p);
}

void ModelAwarePlan::Reset(int64_t batch_size, int64_t seq_len, int64_t num_head, int64_t hidden_size, int64_t num_layer) {
  const std::vector<TensorRecord> records = BertTensorUsageRecords(batch_size, seq_len, num_head, hidden_size, num_layer);
  std::vector<Placement> placements;
  std::vector<bool> used;
  std::vector<int64_t> sizes = chunk_sizes_;
  ChunkedGreedyBySizeOffsetCalculation(records, &sizes, &placements, &used);
  // materialise: keep used old chunks, allocate new ones, release the unused
  std::vector<int> remap(sizes.size(), -1);
  std::vector<int64_t> new_sizes;
  std::vector<void*> new_mem;
  for (size_t c = 0; c < sizes.size(); ++c) {
    const bool existed = c < chunk_mem_.size();
    if (!used[c]) {
      if (existed) free_(chunk_mem_[c]);
      continue;
    }
    void* mem = existed ? chunk_mem_[c] : alloc_((size_t)sizes[c]);
    TT_ENFORCE(mem != nullptr, "model-aware allocator: cannot allocate a chunk of %lld bytes", (long long)sizes[c]);
    remap[c] = (int)new_sizes.size();
    new_sizes.push_back(sizes[c]);
    new_mem.push_back(mem);
  }
  chunk_sizes_.swap(new_sizes);
  chunk_mem_.swap(new_mem);
  position_.clear();
  for (size_t i = 0; i < records.size(); ++i)
    position_[records[i].name] = Position{remap[placements[i].chunk], placements[i].offset, records[i].size};
}

void* ModelAwarePlan::Address(const std::string& name, size_t size) const {
  auto it = position_.find(name);
  TT_ENFORCE(it != position_.end(), "ModelAwareAllocator allocate %s failed", name.c_str());
  TT_ENFORCE((int64_t)size <= it->second.size,
             "model-aware allocator: %s needs %zu bytes but %lld were planned; call bert_opt_mem_allocate_api with the "
             "shape of this input first",
             name.c_str(), size, (long long)it->second.size);
  return static_cast<char*>(chunk_mem_[it->second.chunk]) + it->second.offset;
}

int64_t ModelAwarePlan::chunk_bytes() const { return std::accumulate(chunk_sizes_.begin(), chunk_sizes_.end(), (int64_t)0); }

}  // namespace allocator
}  // namespace core
}  // namespace turbo_transformers
