#include "runner.h"

#include "../host/rules.h"

#include <algorithm>
#include <cstring>

namespace vosti {

// ------------------------------------------------------------------------------------------- pool
static Tensor zeroed(std::vector<int64_t> shape, DType t) {
  Tensor out;
  out.dtype = t;
  out.shape = std::move(shape);
  out.owner = std::make_shared<DeviceBuffer>(out.bytes());
  out.data = out.owner->data();
  hip_check(hipMemset(out.data, 0, out.bytes()), "clearing the cache");
  return out;
}

CachePool::CachePool(DecoderModel& model, int page_size_, int num_pages, int num_slots, bool prefix_cache) : page_size(page_size_) {
  if (page_size < 8 || (page_size & (page_size - 1))) throw EngineError("page size " + std::to_string(page_size) + " must be a power of two, at least 8");
  const std::vector<CacheNeed> needs = model.cache_needs();
  for (const CacheNeed& n : needs) {
    if (n.kind == CacheNeed::Pages && std::find(group_windows.begin(), group_windows.end(), n.window) == group_windows.end())
      group_windows.push_back(n.window);
    if (n.kind == CacheNeed::State) has_state = true;
  }
  std::sort(group_windows.begin(), group_windows.end());     // 0 (all keys) first
  if (group_windows.empty()) group_windows.push_back(0);
  std::vector<GroupSpec> groups;
  for (int w : group_windows) groups.push_back({w, num_pages});
  // A prefix page holds keys only; a mixer with state of its own could not resume from it.
  manager_ = std::make_unique<CacheManager>(page_size, groups, num_slots, prefix_cache && !has_state);
  const DType dtype = model.kernels().dtype();
  const auto& schedule = model.spec().schedule;
  for (size_t i = 0; i < schedule.size(); ++i) {
    CacheEntry e;
    const CacheNeed& n = needs[i];
    if (schedule[i].cache_from >= 0) {
      const CacheEntry& src = entries.at(schedule[i].cache_from);
      if (src.kind != CacheNeed::Pages)
        throw EngineError("schedule entry " + std::to_string(i) + " reads the cache of entry " + std::to_string(schedule[i].cache_from) + ", which keeps no pages");
      e = src;
      e.writable = false;
    } else if (n.kind == CacheNeed::Pages) {
      e.kind = CacheNeed::Pages;
      e.group = (int)(std::find(group_windows.begin(), group_windows.end(), n.window) - group_windows.begin());
      e.page_size = page_size;
      e.k = zeroed({num_pages, n.num_kv_heads, page_size, n.head_dim}, dtype);
      e.v = zeroed({num_pages, n.num_kv_heads, n.head_dim, page_size}, dtype);
      bytes_ += e.k.bytes() + e.v.bytes();
    } else if (n.kind == CacheNeed::State) {
      e.kind = CacheNeed::State;
      std::vector<int64_t> shape = {num_slots};
      shape.insert(shape.end(), n.state_shape.begin(), n.state_shape.end());
      e.state = zeroed(shape, n.state_dtype);
      bytes_ += e.state.bytes();
    }
    entries.push_back(e);
  }
}

// ----------------------------------------------------------------------------------------- runner
struct ModelRunner::Captured {
  hipGraph_t graph = nullptr;
  hipGraphExec_t exec = nullptr;
  int32_t* staging = nullptr;                // pinned host twin of `meta`
  std::unique_ptr<DeviceBuffer> meta;        // the device buffer the graph reads
  size_t ints = 0;
  Tensor logits;                             // the graph's output
  Arena::Mark arena_end;                     // the arena's cursor when the recording ended
  hipEvent_t copied = nullptr;               // the last upload from `staging`
  std::shared_ptr<DeviceBuffer> workspace;   // the buffer its launches point into
  std::list<Key>::iterator lru_it;
  ~Captured() {
    if (exec) (void)hipGraphExecDestroy(exec);
    if (graph) (void)hipGraphDestroy(graph);
    if (staging) (void)hipHostFree(staging);
    if (copied) (void)hipEventDestroy(copied);
  }
};

ModelRunner::ModelRunner(DecoderModel& model, CachePool& pool, bool graphs, int max_graphs)
    : model_(model), pool_(pool), k_(model.kernels()), graphs_(graphs && model.replayable()), max_graphs_(std::max(1, max_graphs)) {
  parts_ = model.parts();
  // What the parts want of every step: one provider per distinct kind of per-step arrays.
  std::set<std::string> keys;
  for (Part* p : parts_)
    if (const char* key = p->step_inputs_key())
      if (keys.insert(key).second) providers_.push_back(p);
  hip_check(hipEventCreateWithFlags(&copied_, hipEventDisableTiming), "event creation");
}

ModelRunner::~ModelRunner() {
  (void)hipStreamSynchronize(k_.stream);
  captured_.clear();
  if (staging_) (void)hipHostFree(staging_);
  if (copied_) (void)hipEventDestroy(copied_);
}

Tensor ModelRunner::workspace(int64_t floats) {
  if (!workspace_ || (int64_t)(workspace_->bytes() / sizeof(float)) < floats) {
    if (capturing_) throw EngineError("a part asks for more workspace inside a recording than it announced before it");
    // Recorded graphs keep the buffer they were recorded with.
    workspace_ = std::make_shared<DeviceBuffer>(sizeof(float) * (size_t)std::max<int64_t>(floats, 1 << 16));
  }
  Tensor t;
  t.data = workspace_->data();
  t.owner = workspace_;          // a part may hold this across a later, larger request: the buffer lives as long as the tensor
  t.dtype = DType::F32;
  t.shape = {(int64_t)(workspace_->bytes() / sizeof(float))};
  return t;
}

int64_t ModelRunner::workspace_needed(HostStep& host) {
  int64_t n = 0;
  for (Part* p : parts_) n = std::max(n, p->workspace_floats(host));
  return n;
}

std::vector<int> ModelRunner::needed_widths(const std::vector<StepEntry>& entries) {
  CacheManager& cache = pool_.manager();
  std::vector<int> w(pool_.group_windows.size(), 1);
  for (const StepEntry& e : entries) {
    if (!cache.has_request(e.id)) throw EngineError("request " + std::to_string(e.id) + " is unknown to the cache");
    for (size_t g = 0; g < w.size(); ++g) w[g] = std::max(w[g], cache.num_logical_pages(e.id, (int)g));
  }
  return w;
}

// The step's host arrays.  widths: block-table width per group (default: what the step needs).  rows: fill up
// to this many sequences with padding rows of one token: token 0 at position 0, one key (whatever page 0
// holds), slot -1 (nothing is stored), logits wanted like the others.  bound > 0: the step is recorded for
// replay and its launches must cover this many keys.
ModelRunner::Layout ModelRunner::layout(const std::vector<StepEntry>& entries, const std::vector<int>* widths, int rows, int bound) {
  CacheManager& cache = pool_.manager();
  const ModelSpec& spec = model_.spec();
  const int real = (int)entries.size();
  const int S = std::max(real, rows), pad = S - real;
  Layout lay;
  HostStep& host = lay.host;
  int T = pad;
  for (const StepEntry& e : entries) {
    if (e.tokens.empty()) throw EngineError("request " + std::to_string(e.id) + ": a step entry needs at least one token");
    if (!cache.has_request(e.id)) throw EngineError("request " + std::to_string(e.id) + " is unknown to the cache");
    const int n = (int)e.tokens.size();
    if (cache.pending(e.id) != n)
      throw EngineError("request " + std::to_string(e.id) + ": the cache holds pages for " + std::to_string(cache.pending(e.id)) +
                        " pending tokens, the step brings " + std::to_string(n));
    host.q_lens.push_back(n);
    host.starts.push_back(cache.length(e.id));
    host.k_lens.push_back(cache.length(e.id) + n);
    host.state_slots.push_back(cache.state_slot(e.id));
    T += n;
  }
  for (int i = 0; i < pad; ++i) {
    host.q_lens.push_back(1);
    host.starts.push_back(0);
    host.k_lens.push_back(1);
    host.state_slots.push_back(0);
  }
  const int longest = *std::max_element(host.k_lens.begin(), host.k_lens.end());
  if (longest > spec.max_positions)
    throw EngineError("a request would reach " + std::to_string(longest) + " tokens; the model's positions end at " + std::to_string(spec.max_positions));
  host.k_len_bound = bound > 0 ? bound : longest;
  host.frozen = bound > 0;

  std::vector<HostArray> arrays(6);
  HostArray &ids = arrays[0], &positions = arrays[1], &cu_q = arrays[2], &k_len = arrays[3], &slots = arrays[4], &want = arrays[5];
  cu_q.data.push_back(0);
  for (int s = 0; s < S; ++s) {
    const int base = cu_q.data.back();
    if (s < real) {
      for (int32_t t : entries[s].tokens) {
        if (t < 0 || t >= spec.vocab_size) throw EngineError("token id out of range [0, " + std::to_string(spec.vocab_size) + ")");
        ids.data.push_back(t);
      }
      for (int w : entries[s].want) {
        if (w < 0 || w >= host.q_lens[s])
          throw EngineError("request " + std::to_string(entries[s].id) + ": wanted place " + std::to_string(w) + " is outside its " +
                            std::to_string(host.q_lens[s]) + " tokens");
        want.data.push_back(base + w);
      }
    } else {
      ids.data.push_back(0);
      want.data.push_back(base);
    }
    for (int i = 0; i < host.q_lens[s]; ++i) positions.data.push_back(host.starts[s] + i);
    cu_q.data.push_back(base + host.q_lens[s]);
    k_len.data.push_back(host.k_lens[s]);
    slots.data.push_back(host.state_slots[s]);
  }
  ids.shape = positions.shape = {T};
  cu_q.shape = {S + 1};
  k_len.shape = slots.shape = {S};
  want.shape = {(int64_t)want.data.size()};
  lay.wanted = (int)want.data.size();
  const std::vector<int> needed = widths ? *widths : needed_widths(entries);
  for (size_t g = 0; g < pool_.group_windows.size(); ++g) {
    const int width = needed[g];
    HostArray sl, table;
    sl.data.assign(T, -1);
    sl.shape = {T};
    table.data.assign((size_t)S * width, 0);
    table.shape = {S, width};
    int at = 0;
    for (int s = 0; s < real; ++s) {
      if (cache.fill_block_table(entries[s].id, (int)g, table.data.data() + (size_t)s * width, width) != OK ||
          cache.fill_slots(entries[s].id, (int)g, host.starts[s], host.q_lens[s], sl.data.data() + at) != OK)
        throw EngineError("request " + std::to_string(entries[s].id) + ": the cache manager could not describe its pages");
      at += host.q_lens[s];
    }
    arrays.push_back(std::move(sl));
    arrays.push_back(std::move(table));
  }
  for (Part* provider : providers_) {
    std::vector<std::pair<std::string, HostArray>> out;
    provider->step_inputs(host, out);
    for (auto& na : out) {
      if (std::find(lay.names.begin(), lay.names.end(), na.first) != lay.names.end())
        throw EngineError("two parts ask for a per-step array named '" + na.first + "'");
      lay.names.push_back(na.first);
      arrays.push_back(std::move(na.second));
    }
  }
  // One buffer, one copy; every piece starts on a 16-byte boundary.
  size_t total = 0;
  for (const HostArray& a : arrays) {
    lay.pieces.push_back({total, a.shape});
    total += (a.data.size() + 3) & ~(size_t)3;
  }
  lay.buf.assign(std::max<size_t>(total, 4), 0);
  for (size_t i = 0; i < arrays.size(); ++i)
    if (!arrays[i].data.empty()) std::memcpy(lay.buf.data() + lay.pieces[i].offset, arrays[i].data.data(), arrays[i].data.size() * sizeof(int32_t));
  return lay;
}

// Runs the model on a layout whose numbers lie at meta_dev.
Tensor ModelRunner::forward(Layout& lay, int32_t* meta_dev) {
  auto view = [&](size_t i) {
    Tensor t;
    t.data = meta_dev + lay.pieces[i].offset;
    t.dtype = DType::I32;
    t.shape = lay.pieces[i].shape;
    return t;
  };
  StepContext ctx;
  ctx.kernels = &k_;
  ctx.num_seqs = (int)lay.host.q_lens.size();
  ctx.num_tokens = (int)lay.pieces[0].shape[0];
  ctx.positions = view(1);
  ctx.cu_q = view(2);
  ctx.k_len = view(3);
  ctx.state_slots = view(4);
  const size_t G = pool_.group_windows.size();
  for (size_t g = 0; g < G; ++g) ctx.groups.push_back({view(6 + 2 * g), view(7 + 2 * g), pool_.group_windows[g]});
  for (size_t i = 0; i < lay.names.size(); ++i) ctx.inputs[lay.names[i]] = view(6 + 2 * G + i);
  ctx.host = &lay.host;
  ctx.workspace = [this](int64_t n) { return workspace(n); };
  k_.arena.reset();
  return model_.forward(view(0), ctx, pool_.entries, view(5));
}

Tensor ModelRunner::run_eager(const std::vector<StepEntry>& entries) {
  ++stats_.eager;
  Layout lay = layout(entries, nullptr, 0, 0);
  if (lay.buf.size() > staging_ints_) {
    hip_check(hipStreamSynchronize(k_.stream), "waiting for the stream");
    if (staging_) (void)hipHostFree(staging_);
    staging_ints_ = std::max<size_t>(2 * lay.buf.size(), 1 << 14);
    hip_check(hipHostMalloc(reinterpret_cast<void**>(&staging_), staging_ints_ * sizeof(int32_t), hipHostMallocDefault), "pinned allocation");
    meta_ = std::make_unique<DeviceBuffer>(staging_ints_ * sizeof(int32_t));
  }
  hip_check(hipEventSynchronize(copied_), "waiting for the last upload");      // the staging buffer is free again
  std::memcpy(staging_, lay.buf.data(), lay.buf.size() * sizeof(int32_t));
  hip_check(hipMemcpyAsync(meta_->data(), staging_, lay.buf.size() * sizeof(int32_t), hipMemcpyHostToDevice, k_.stream), "step upload");
  hip_check(hipEventRecord(copied_, k_.stream), "event record");
  // What the parts announced, before the first of them runs: a part that asks twice in its forward (a projection's
  // chunk sums, then the attention's partial results) then gets the same buffer both times.
  workspace(workspace_needed(lay.host));
  return forward(lay, static_cast<int32_t*>(meta_->data()));
}

void ModelRunner::drop_captured() {
  (void)hipStreamSynchronize(k_.stream);
  captured_.clear();
  lru_.clear();
}

ModelRunner::Captured* ModelRunner::capture(const Key& key, Layout& lay) {
  while ((int)captured_.size() >= max_graphs_) {     // the least recently replayed goes first
    hip_check(hipStreamSynchronize(k_.stream), "waiting for the stream");
    captured_.erase(lru_.front());
    lru_.pop_front();
    ++stats_.evicted;
  }
  auto cap = std::make_unique<Captured>();
  cap->ints = lay.buf.size();
  hip_check(hipHostMalloc(reinterpret_cast<void**>(&cap->staging), cap->ints * sizeof(int32_t), hipHostMallocDefault), "pinned allocation");
  cap->meta = std::make_unique<DeviceBuffer>(cap->ints * sizeof(int32_t));
  hip_check(hipEventCreateWithFlags(&cap->copied, hipEventDisableTiming), "event creation");
  std::memcpy(cap->staging, lay.buf.data(), cap->ints * sizeof(int32_t));
  hip_check(hipMemcpyAsync(cap->meta->data(), cap->staging, cap->ints * sizeof(int32_t), hipMemcpyHostToDevice, k_.stream), "step upload");
  workspace(workspace_needed(lay.host));
  cap->workspace = workspace_;
  int32_t* meta = static_cast<int32_t*>(cap->meta->data());
  // Once outside a recording: the arena grows to what the step needs, and every kernel has run once.
  forward(lay, meta);
  hip_check(hipStreamSynchronize(k_.stream), "the step before its recording");
  capturing_ = true;
  k_.arena.forbid_growth(true);
  hipError_t begun = hipStreamBeginCapture(k_.stream, hipStreamCaptureModeThreadLocal);
  try {
    hip_check(begun, "begin of the recording");
    cap->logits = forward(lay, meta);
    cap->arena_end = k_.arena.mark();
    hip_check(hipStreamEndCapture(k_.stream, &cap->graph), "end of the recording");
  } catch (...) {
    if (begun == hipSuccess && !cap->graph) {
      hipGraph_t broken = nullptr;
      (void)hipStreamEndCapture(k_.stream, &broken);
      if (broken) (void)hipGraphDestroy(broken);
    }
    capturing_ = false;
    k_.arena.forbid_growth(false);
    throw;
  }
  capturing_ = false;
  k_.arena.forbid_growth(false);
  hip_check(hipGraphInstantiate(&cap->exec, cap->graph, nullptr, nullptr, 0), "graph instantiation");
  lru_.push_back(key);
  cap->lru_it = std::prev(lru_.end());
  Captured* raw = cap.get();
  captured_[key] = std::move(cap);
  ++stats_.captured;
  return raw;
}

Tensor ModelRunner::run_decode_graph(const std::vector<StepEntry>& entries) {
  if (!poisoned_.empty()) throw GraphError("graph replay is switched off after a failure: " + poisoned_);
  std::vector<int> widths = needed_widths(entries);
  for (int& w : widths) w = graph_width_bucket(w);
  // A mixer with state of its own would have to be told which rows are padding: no padding then.
  const int rows = pool_.has_state ? (int)entries.size() : graph_row_bucket((int)entries.size());
  const Key key{rows, widths};
  auto it = captured_.find(key);
  if (it == captured_.end() && seen_.insert(key).second) return run_eager(entries);   // first sight of a signature
  // Launch geometry is frozen in the graph: it must cover every length the tables can hold.
  const int cover = (int)std::min<int64_t>((int64_t)*std::max_element(widths.begin(), widths.end()) * pool_.page_size, model_.spec().max_positions);
  Tensor logits;
  try {
    Layout lay = layout(entries, &widths, rows, cover);
    Captured* cap;
    if (it == captured_.end()) {
      cap = capture(key, lay);
    } else {
      cap = it->second.get();
      lru_.splice(lru_.end(), lru_, cap->lru_it);
      if (lay.buf.size() != cap->ints) throw EngineError("a step's numbers do not fit the recording of its signature");
      hip_check(hipEventSynchronize(cap->copied), "waiting for the last upload");
      std::memcpy(cap->staging, lay.buf.data(), cap->ints * sizeof(int32_t));
      hip_check(hipMemcpyAsync(cap->meta->data(), cap->staging, cap->ints * sizeof(int32_t), hipMemcpyHostToDevice, k_.stream), "step upload");
    }
    hip_check(hipEventRecord(cap->copied, k_.stream), "event record");
    hip_check(hipGraphLaunch(cap->exec, k_.stream), "graph launch");
    // No forward() ran, so the arena's cursor is wherever the last eager step left it, which may be in the
    // middle of this recording's results.
    k_.arena.restore(cap->arena_end);
    logits = cap->logits.rows(0, (int64_t)entries.size());
  } catch (const std::exception& e) {
    poisoned_ = e.what();
    drop_captured();
    throw GraphError("graph recording or replay failed (" + poisoned_ + "); no further step is replayed");
  }
  ++stats_.replayed;
  return logits;
}

Tensor ModelRunner::run(const std::vector<StepEntry>& entries) {
  bool decode_only = graphs_;
  for (const StepEntry& e : entries) decode_only = decode_only && e.tokens.size() == 1 && e.want.size() == 1 && e.want[0] == 0;
  return decode_only ? run_decode_graph(entries) : run_eager(entries);
}

Tensor ModelRunner::step(const std::vector<StepEntry>& entries) {
  if (entries.empty()) return k_.empty({0, model_.spec().vocab_size});
  CacheManager& cache = pool_.manager();
  std::set<RequestId> ids;
  for (const StepEntry& e : entries)
    if (!ids.insert(e.id).second) throw EngineError("a request appears twice in one step");
  std::vector<RequestId> taken;
  auto give_up = [&] {
    for (RequestId id : taken) cache.abort_step(id);
  };
  try {
    for (const StepEntry& e : entries) {
      if (e.tokens.empty()) throw EngineError("request " + std::to_string(e.id) + ": a step entry needs at least one token");
      if (!cache.has_request(e.id)) {
        const Status st = cache.add_request(e.id, nullptr, 0, nullptr);
        if (st != OK) throw EngineError("request " + std::to_string(e.id) + ": no state slot is free");
      }
      const Status st = cache.extend(e.id, e.tokens.data(), (int)e.tokens.size());
      if (st != OK) throw EngineError("request " + std::to_string(e.id) + (st == NO_PAGES ? ": out of cache pages" : ": the cache manager refused its tokens"));
      taken.push_back(e.id);
    }
    Tensor logits = run(entries);
    for (const StepEntry& e : entries) cache.commit(e.id);
    return logits;
  } catch (...) {
    give_up();
    throw;
  }
}

void ModelRunner::finish(RequestId id) { pool_.manager().finish(id); }

}  // namespace vosti
