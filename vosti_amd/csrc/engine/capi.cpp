// The native engine as a library: a C interface over Engine for callers in other languages (the Python
// package's NativeEngine drives it through ctypes).  Every function that can fail returns -1 (or null)
// and leaves the reason in the caller's buffer; nothing throws across the boundary.
#include <cstring>

#include "engine.h"

using namespace vosti;

namespace {
void put(char* err, int cap, const std::string& text) {
  if (!err || cap <= 0) return;
  std::strncpy(err, text.c_str(), (size_t)cap - 1);
  err[cap - 1] = 0;
}
}  // namespace

extern "C" {

int ve_abi_version(void) { return 3; }

// Loads a shared library of part kinds and architectures (load_plugin in parts.h).  0, or -1 with the reason.
int ve_load_plugin(const char* path, char* err, int errcap) {
  try {
    load_plugin(path);
    return 0;
  } catch (const std::exception& e) {
    put(err, errcap, e.what());
    return -1;
  }
}

// 1 if this library can run the model in the folder; 0 if its architecture or one of its part kinds is not
// registered here (err says which); -1 if config.json is missing or breaks a rule (err says how).
int ve_supports(const char* model_dir, char* err, int errcap) {
  try {
    const std::string why = why_unsupported(model_dir);
    if (why.empty()) return 1;
    put(err, errcap, why);
    return 0;
  } catch (const std::exception& e) {
    put(err, errcap, e.what());
    return -1;
  }
}

// dtype: "bf16" or "f32".  random_weights != 0: the folder needs config.json only and the weights are drawn
// from `seed` on the GPU.
void* ve_create(const char* model_dir, const char* lib_dir, const char* dtype, int num_pages, int page_size, int max_num_seqs,
                int max_num_batched_tokens, int prefix_cache, int max_model_len, int graphs, int random_weights, uint64_t seed,
                char* err, int errcap) {
  try {
    EngineOptions o;
    o.model_dir = model_dir;
    o.lib_dir = lib_dir;
    o.dtype = dtype;
    o.num_pages = num_pages;
    o.page_size = page_size;
    o.max_num_seqs = max_num_seqs;
    o.max_num_batched_tokens = max_num_batched_tokens;
    o.prefix_cache = prefix_cache != 0;
    o.max_model_len = max_model_len;
    o.graphs = graphs != 0;
    o.random_weights = random_weights != 0;
    o.random_seed = seed;
    return new Engine(o);
  } catch (const std::exception& e) {
    put(err, errcap, e.what());
    return nullptr;
  }
}

void ve_destroy(void* h) { delete static_cast<Engine*>(h); }

// Returns the request's id, or -1.
int64_t ve_add_request(void* h, const int32_t* prompt, int n_prompt, int max_tokens, float temperature, uint64_t seed,
                       const int32_t* eos, int n_eos, int ignore_eos, char* err, int errcap) {
  try {
    SamplingParams p;
    p.max_tokens = max_tokens;
    p.temperature = temperature;
    p.seed = seed;
    p.eos_token_ids.assign(eos, eos + (n_eos > 0 ? n_eos : 0));
    p.ignore_eos = ignore_eos != 0;
    return (int64_t) static_cast<Engine*>(h)->add_request(std::vector<int32_t>(prompt, prompt + (n_prompt > 0 ? n_prompt : 0)), p);
  } catch (const std::exception& e) {
    put(err, errcap, e.what());
    return -1;
  }
}

// One engine step.  out: pairs (request id, emitted token), room for `cap` of them.  Returns their number, or -1.
int ve_step(void* h, int64_t* out, int cap, char* err, int errcap) {
  try {
    const auto emitted = static_cast<Engine*>(h)->step();
    if ((int)emitted.size() > cap) throw EngineError("more tokens emitted than the caller has room for");
    for (size_t i = 0; i < emitted.size(); ++i) {
      out[2 * i] = (int64_t)emitted[i].first;
      out[2 * i + 1] = emitted[i].second;
    }
    return (int)emitted.size();
  } catch (const std::exception& e) {
    put(err, errcap, e.what());
    return -1;
  }
}

int ve_has_unfinished(void* h) { return static_cast<Engine*>(h)->has_unfinished() ? 1 : 0; }

int ve_synchronize(void* h, char* err, int errcap) {
  try {
    static_cast<Engine*>(h)->synchronize();
    return 0;
  } catch (const std::exception& e) {
    put(err, errcap, e.what());
    return -1;
  }
}

// out[0..3]: graph steps run eagerly, recorded, replayed, recordings dropped; out[4], out[5]: admissions that
// found a cached prefix and the pages they found; out[6]: preemptions; out[7]: requests the cache manager holds;
// out[8]: vocabulary size; out[9]: positions of the model.
void ve_stats(void* h, int64_t* out) {
  Engine* e = static_cast<Engine*>(h);
  const GraphStats& g = e->runner().graph_stats();
  out[0] = g.eager; out[1] = g.captured; out[2] = g.replayed; out[3] = g.evicted;
  out[4] = e->cache().prefix_hit_requests();
  out[5] = e->cache().prefix_hits();
  out[6] = e->scheduler().preemptions();
  out[7] = e->cache().num_requests();
  out[8] = e->model().spec().vocab_size;
  out[9] = e->model().spec().max_positions;
}

// ---- The step function alone, for replaying given tokens (no scheduler, no sampling).  An engine is used either
// this way or through ve_add_request / ve_step, not both: the two share the cache manager.

// Announces a request's whole prompt so that cached pages can be matched (with the prefix cache on).  Returns the
// number of its first tokens that are cached already, or -1.
int ve_trace_add_request(void* h, int64_t id, const int32_t* prompt, int n_prompt, char* err, int errcap) {
  try {
    int cached = 0;
    const Status st = static_cast<Engine*>(h)->cache().add_request((RequestId)id, prompt, n_prompt, &cached);
    if (st != OK) throw EngineError("request " + std::to_string(id) + " was refused by the cache manager (status " + std::to_string((int)st) + ")");
    return cached;
  } catch (const std::exception& e) {
    put(err, errcap, e.what());
    return -1;
  }
}

// One step: entry i is request ids[i] with the next tokens[tok_off[i] .. tok_off[i + 1]) and the wanted places
// want[want_off[i] .. want_off[i + 1]) among them.  The logits at the wanted places, in the order of the entries and
// of `want`, go to `out` as float32 [wanted, vocabulary] (room for out_floats).  Returns the wanted rows, or -1.
int64_t ve_trace_step(void* h, int n_entries, const int64_t* ids, const int32_t* tok_off, const int32_t* tokens,
                      const int32_t* want_off, const int32_t* want, float* out, int64_t out_floats, char* err, int errcap) {
  try {
    Engine* e = static_cast<Engine*>(h);
    std::vector<StepEntry> entries((size_t)(n_entries > 0 ? n_entries : 0));
    for (int i = 0; i < n_entries; ++i) {
      entries[i].id = (RequestId)ids[i];
      entries[i].tokens.assign(tokens + tok_off[i], tokens + tok_off[i + 1]);
      entries[i].want.assign(want + want_off[i], want + want_off[i + 1]);
    }
    const Tensor logits = e->runner().step(entries);
    const int64_t rows = logits.numel() ? logits.dim(0) : 0;
    if (rows > 0) {
      if (logits.numel() > out_floats) throw EngineError("the caller's buffer is too small for the wanted logits");
      Kernels& k = e->model().kernels();
      const Tensor f = k.to_f32(logits);
      hip_check(hipMemcpyAsync(out, f.data, f.bytes(), hipMemcpyDeviceToHost, k.stream), "logits readback");
    }
    e->synchronize();
    return rows;
  } catch (const std::exception& e) {
    put(err, errcap, e.what());
    return -1;
  }
}

int ve_trace_has_request(void* h, int64_t id) { return static_cast<Engine*>(h)->cache().has_request((RequestId)id) ? 1 : 0; }

// The request is over: what it holds is given back.
int ve_trace_finish(void* h, int64_t id, char* err, int errcap) {
  try {
    static_cast<Engine*>(h)->runner().finish((RequestId)id);
    return 0;
  } catch (const std::exception& e) {
    put(err, errcap, e.what());
    return -1;
  }
}

// Writes the cache manager's first violated invariant into buf (empty if none); returns its length.
int ve_cache_check(void* h, char* buf, int cap) {
  const std::string s = static_cast<Engine*>(h)->cache().check();
  put(buf, cap, s);
  return (int)s.size();
}

}  // extern "C"
