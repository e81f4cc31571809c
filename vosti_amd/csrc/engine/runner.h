// The tensors behind the cache manager's numbers, and the step function: one batch of (request, its next
// tokens) through the model.
//
// A step runs only the tokens it is given, from the cache that earlier steps left: portions of prompts
// beside single decoded tokens, cut anywhere.  It returns the logits at the places that are asked for.
// The reference's counterpart is model_forward with the six step tensors (src/exec/model.rs:62-85,
// src/exec/cache_scheduler/mod.rs:824-930); here the wanted rows are arbitrary, not only each sequence's last.
//
// Steps that hold nothing but single decoded tokens, each wanting its logits, can be replayed from a
// recorded HIP graph: the same forward pass, recorded once per (number of rows, block-table widths) and fed
// through fixed device buffers.  The reference does the same around its forward
// (python/vosti_kernels/graph_overlay.py:177-389): a signature runs eagerly when first seen, is recorded
// when seen again, and is replayed from then on.
#pragma once
#include <list>
#include <map>
#include <memory>
#include <set>
#include <string>
#include <vector>

#include "../host/cache_manager.h"
#include "../host/rules.h"
#include "model.h"

namespace vosti {

// A recording or a replay failed: the runner replays nothing any more
// (python/vosti_kernels/graph_overlay.py:120-124, 173-175: no eager fallback after a failed replay).
struct GraphError : EngineError {
  using EngineError::EngineError;
};

class CachePool {
 public:
  // num_pages: pages of every group.  One group per distinct window; every all-keys layer shares group 0's
  // page numbers, as in the reference where one block id names the same page in every layer
  // (python/vosti_kernels/physical.py:139-147).
  CachePool(DecoderModel& model, int page_size, int num_pages, int num_slots, bool prefix_cache);
  CacheManager& manager() { return *manager_; }
  std::vector<CacheEntry> entries;          // one per schedule entry
  std::vector<int> group_windows;
  int page_size;
  bool has_state = false;
  size_t bytes() const { return bytes_; }

 private:
  std::unique_ptr<CacheManager> manager_;
  size_t bytes_ = 0;
};

struct StepEntry {
  RequestId id = 0;
  std::vector<int32_t> tokens;
  std::vector<int> want;                    // places among `tokens` whose logits are wanted
};

struct GraphStats {
  int64_t eager = 0, captured = 0, replayed = 0, evicted = 0;
};

class ModelRunner {
 public:
  ModelRunner(DecoderModel& model, CachePool& pool, bool graphs, int max_graphs = kMaxGraphs);
  ~ModelRunner();

  // The forward pass of a step whose pages are taken; logits [wanted, vocab] in the element type, valid
  // until the next call.
  Tensor run(const std::vector<StepEntry>& entries);
  // Pages, forward, commit, for callers without a scheduler.
  Tensor step(const std::vector<StepEntry>& entries);
  void finish(RequestId id);
  const GraphStats& graph_stats() const { return stats_; }

 private:
  struct Piece {
    size_t offset = 0;
    std::vector<int64_t> shape;
  };
  struct Layout {
    std::vector<int32_t> buf;               // every array of the step, each on a 16-byte boundary
    std::vector<Piece> pieces;              // ids, positions, cu_q, k_len, state slots, wanted rows, (slots, table) per group, then parts' arrays
    std::vector<std::string> names;         // of the parts' arrays
    HostStep host;
    int wanted = 0;
  };
  struct Captured;
  using Key = std::pair<int, std::vector<int>>;

  Layout layout(const std::vector<StepEntry>& entries, const std::vector<int>* widths, int rows, int bound);
  std::vector<int> needed_widths(const std::vector<StepEntry>& entries);
  Tensor forward(Layout& lay, int32_t* meta_dev);
  Tensor run_eager(const std::vector<StepEntry>& entries);
  Tensor run_decode_graph(const std::vector<StepEntry>& entries);
  Captured* capture(const Key& key, Layout& lay);
  Tensor workspace(int64_t floats);
  int64_t workspace_needed(HostStep& host);
  void drop_captured();

  DecoderModel& model_;
  CachePool& pool_;
  Kernels& k_;
  bool graphs_;
  int max_graphs_;
  std::vector<Part*> parts_;
  std::vector<Part*> providers_;
  std::shared_ptr<DeviceBuffer> workspace_;
  bool capturing_ = false;
  // Eager steps' upload buffers.
  int32_t* staging_ = nullptr;              // pinned
  std::unique_ptr<DeviceBuffer> meta_;
  size_t staging_ints_ = 0;
  hipEvent_t copied_ = nullptr;
  std::set<Key> seen_;
  std::map<Key, std::unique_ptr<Captured>> captured_;
  std::list<Key> lru_;                      // least recently replayed first
  std::string poisoned_;
  GraphStats stats_;
};

}  // namespace vosti
