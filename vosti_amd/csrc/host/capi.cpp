// C interface of the host library, for ctypes.
#include <cstring>
#include <string>
#include <vector>

#include "cache_manager.h"
#include "rules.h"
#include "scheduler.h"
#include "spec.h"

using namespace vosti;

namespace {
struct SchedulerHandle {
  Scheduler sched;
  std::vector<PlanRow> rows;
  std::vector<int32_t> tokens;
  std::vector<Emitted> emitted;
  SchedulerHandle(CacheManager* c, SchedulerConfig cfg) : sched(c, cfg) {}
};
}  // namespace

extern "C" {

int vh_abi_version(void) { return 8; }

// ------------------------------------------------------------ cache manager
void* vh_cache_create(int page_size, int n_groups, const int* windows, const int* num_pages, int num_slots,
                      int prefix_cache) {
  if (page_size <= 0 || n_groups <= 0 || num_slots < 0) return nullptr;
  std::vector<GroupSpec> groups;
  for (int g = 0; g < n_groups; ++g) {
    if (windows[g] < 0 || num_pages[g] < 0) return nullptr;
    groups.push_back(GroupSpec{windows[g], num_pages[g]});
  }
  return new CacheManager(page_size, groups, num_slots, prefix_cache != 0);
}
void vh_cache_destroy(void* h) { delete static_cast<CacheManager*>(h); }

#define CM static_cast<CacheManager*>(h)
int vh_cache_add_request(void* h, uint64_t id, const int32_t* prompt, int n, int* cached) {
  return CM->add_request(id, prompt, n, cached);
}
int vh_cache_reserve(void* h, uint64_t id, int total) { return CM->reserve(id, total); }
int vh_cache_extend(void* h, uint64_t id, const int32_t* tokens, int n) { return CM->extend(id, tokens, n); }
int vh_cache_commit(void* h, uint64_t id) { return CM->commit(id); }
int vh_cache_abort_step(void* h, uint64_t id) { return CM->abort_step(id); }
int vh_cache_finish(void* h, uint64_t id) { return CM->finish(id); }
int vh_cache_has_request(void* h, uint64_t id) { return CM->has_request(id) ? 1 : 0; }
int vh_cache_length(void* h, uint64_t id) { return CM->length(id); }
int vh_cache_pending(void* h, uint64_t id) { return CM->pending(id); }
int vh_cache_state_slot(void* h, uint64_t id) { return CM->state_slot(id); }
int vh_cache_num_logical_pages(void* h, uint64_t id, int g) { return CM->num_logical_pages(id, g); }
int vh_cache_available_pages(void* h, int g) { return CM->available_pages(g); }
int vh_cache_free_pages(void* h, int g) { return CM->free_pages(g); }
int vh_cache_free_slots(void* h) { return CM->free_slots(); }
int vh_cache_num_requests(void* h) { return CM->num_requests(); }
int vh_cache_cached_blocks(void* h) { return CM->cached_blocks(); }
int vh_cache_drop_cached(void* h) { return CM->drop_cached(); }
int64_t vh_cache_prefix_hits(void* h) { return CM->prefix_hits(); }
int64_t vh_cache_prefix_hit_requests(void* h) { return CM->prefix_hit_requests(); }
int64_t vh_cache_evictions(void* h) { return CM->evictions(); }
int vh_cache_fill_block_table(void* h, uint64_t id, int g, int32_t* out, int width) {
  return CM->fill_block_table(id, g, out, width);
}
int vh_cache_fill_slots(void* h, uint64_t id, int g, int start, int n, int32_t* out) {
  return CM->fill_slots(id, g, start, n, out);
}
// What a step needs to know of its n requests, in one call: per request its committed length, its
// pending tokens and its state slot (out: n x 3), and per request and group the block-table width it
// needs (widths: n x n_groups).  Returns OK or the first request's error.
int vh_cache_describe(void* h, int n, const uint64_t* ids, int32_t* out, int32_t* widths) {
  const int G = CM->num_groups();
  for (int i = 0; i < n; ++i) {
    if (!CM->has_request(ids[i])) return UNKNOWN_REQUEST;
    out[3 * i] = CM->length(ids[i]);
    out[3 * i + 1] = CM->pending(ids[i]);
    out[3 * i + 2] = CM->state_slot(ids[i]);
    for (int g = 0; g < G; ++g) widths[i * G + g] = CM->num_logical_pages(ids[i], g);
  }
  return OK;
}
// The block table [rows, width] (rows beyond n, and entries beyond a request's pages, read page 0) and
// the slots of every token of the step (n_tokens[i] tokens from starts[i] on; slots has room for their
// sum plus `pad_tokens` entries, which get -1) of one group.
int vh_cache_fill_step(void* h, int group, int n, const uint64_t* ids, const int32_t* starts, const int32_t* n_tokens,
                       int rows, int width, int32_t* table, int pad_tokens, int32_t* slots) {
  int64_t t = 0;
  for (int i = 0; i < n; ++i) {
    Status st = CM->fill_block_table(ids[i], group, table + (int64_t)i * width, width);
    if (st != OK) return st;
    st = CM->fill_slots(ids[i], group, starts[i], n_tokens[i], slots + t);
    if (st != OK) return st;
    t += n_tokens[i];
  }
  for (int64_t i = (int64_t)n * width; i < (int64_t)rows * width; ++i) table[i] = 0;
  for (int i = 0; i < pad_tokens; ++i) slots[t + i] = -1;
  return OK;
}
// Writes the first violated invariant into buf (empty if none); returns its length.
int vh_cache_check(void* h, char* buf, int cap) {
  const std::string s = CM->check();
  if (cap > 0) {
    std::strncpy(buf, s.c_str(), cap - 1);
    buf[cap - 1] = 0;
  }
  return (int)s.size();
}
#undef CM

// ---------------------------------------------------------------- scheduler
void* vh_sched_create(void* cache, int max_num_seqs, int max_num_batched_tokens, int max_model_len) {
  if (cache == nullptr || max_num_seqs <= 0 || max_num_batched_tokens <= 0 || max_model_len <= 0) return nullptr;
  return new SchedulerHandle(static_cast<CacheManager*>(cache),
                             SchedulerConfig{max_num_seqs, max_num_batched_tokens, max_model_len});
}
void vh_sched_destroy(void* h) { delete static_cast<SchedulerHandle*>(h); }

#define SH static_cast<SchedulerHandle*>(h)
int vh_sched_add_request(void* h, uint64_t id, const int32_t* prompt, int n_prompt, int max_tokens,
                         const int32_t* eos, int n_eos, int ignore_eos) {
  return SH->sched.add_request(id, prompt, n_prompt, max_tokens, eos, n_eos, ignore_eos != 0);
}
// Returns the plan status; *n_rows and *n_tokens describe the planned step.
int vh_sched_plan(void* h, int* n_rows, int* n_tokens) {
  const int st = SH->sched.plan(SH->rows, SH->tokens);
  *n_rows = (int)SH->rows.size();
  *n_tokens = (int)SH->tokens.size();
  return st;
}
// rows_out: n_rows x 6 int64 (id, start, n_tokens, sample, state_slot, output_index).
void vh_sched_get_plan(void* h, int64_t* rows_out, int32_t* tokens_out) {
  for (size_t i = 0; i < SH->rows.size(); ++i) {
    const PlanRow& r = SH->rows[i];
    int64_t* o = rows_out + 6 * i;
    o[0] = (int64_t)r.id; o[1] = r.start; o[2] = r.n_tokens; o[3] = r.sample; o[4] = r.state_slot; o[5] = r.output_index;
  }
  if (!SH->tokens.empty()) std::memcpy(tokens_out, SH->tokens.data(), SH->tokens.size() * sizeof(int32_t));
}
// Returns the number of emitted tokens, or -1 (nothing committed) if n_sampled is not the number of
// sampled rows of the plan.
int vh_sched_commit(void* h, const int32_t* sampled, int n_sampled) {
  if (!SH->sched.commit(sampled, n_sampled, SH->emitted)) return -1;
  return (int)SH->emitted.size();
}
void vh_sched_abort_step(void* h) { SH->sched.abort_step(); }
int vh_sched_num_planned_samples(void* h) { return SH->sched.num_planned_samples(); }
// out: n x 3 int64 (id, token, finished).
void vh_sched_get_emitted(void* h, int64_t* out) {
  for (size_t i = 0; i < SH->emitted.size(); ++i) {
    out[3 * i] = (int64_t)SH->emitted[i].id;
    out[3 * i + 1] = SH->emitted[i].token;
    out[3 * i + 2] = SH->emitted[i].finished;
  }
}
int vh_sched_abort(void* h, uint64_t id) { return SH->sched.abort(id) ? 1 : 0; }
int vh_sched_num_waiting(void* h) { return SH->sched.num_waiting(); }
int vh_sched_num_running(void* h) { return SH->sched.num_running(); }
int64_t vh_sched_preemptions(void* h) { return SH->sched.preemptions(); }
int vh_sched_is_live(void* h, uint64_t id) { return SH->sched.is_live(id) ? 1 : 0; }
#undef SH

// ------------------------------------------------- configurations and shared rules
// What the architecture named by a config.json's text makes of it: model_spec_json().  Returns the text's
// length (the caller's buffer got it whole if that is below cap), or -1 with the reason in err; -2 if no
// registered architecture is named (err says which are).
int vh_describe_config(const char* config_text, char* out, int cap, char* err, int errcap) {
  auto fail = [&](const std::string& what, int rc) {
    if (err && errcap > 0) {
      std::strncpy(err, what.c_str(), (size_t)errcap - 1);
      err[errcap - 1] = 0;
    }
    return rc;
  };
  try {
    register_builtin_architectures();
    const Json raw = Json::parse(config_text);
    if (!architecture_known(raw)) {
      try {
        model_spec_from_config(raw);
      } catch (const std::exception& e) {
        return fail(e.what(), -2);
      }
    }
    const std::string text = model_spec_json(model_spec_from_config(raw));
    if ((int)text.size() < cap) std::memcpy(out, text.c_str(), text.size() + 1);
    return (int)text.size();
  } catch (const JsonError& e) {
    return fail(std::string("config.json is not valid JSON: ") + e.what(), -1);
  } catch (const std::exception& e) {
    return fail(e.what(), -1);
  }
}

// "model_type=Architecture" lines of every registered architecture.
int vh_model_types(char* out, int cap) {
  register_builtin_architectures();
  std::string text;
  for (const auto& t : model_types()) text += t.first + "=" + t.second + "\n";
  if ((int)text.size() < cap) std::memcpy(out, text.c_str(), text.size() + 1);
  return (int)text.size();
}

void vh_rotary_inverse_frequencies(double theta, int rotary_dim, float* out) { rotary_inverse_frequencies(theta, rotary_dim, out); }
int vh_graph_row_bucket(int rows) { return graph_row_bucket(rows); }
int vh_graph_width_bucket(int pages) { return graph_width_bucket(pages); }
int vh_max_graphs(void) { return kMaxGraphs; }

}  // extern "C"
