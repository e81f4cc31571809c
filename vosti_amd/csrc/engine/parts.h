// The parts a decoder is put together from, as the native engine knows them: the same categories, kinds
// and parameters as the Python package's parts (vosti_amd/parts), chosen by the same descriptions, and the
// same kernels below them.  No part knows which model it is in.
//
// A new kind is one class and one register_part() call; an architecture names it in its description.  Kinds
// and architectures can also come from outside this library: load_plugin() loads a shared library that was
// compiled against these headers and calls its vosti_plugin_register(), which registers what it brings.
#pragma once
#include <functional>
#include <map>
#include <memory>
#include <string>
#include <utility>
#include <vector>

#include "gpu.h"
#include "../host/spec.h"

namespace vosti {

struct ParamDecl {
  std::string name;               // local name, e.g. "q_proj.weight"
  std::vector<int64_t> shape;
  bool keep_f32 = false;          // a tensor the file stores in 32-bit stays so
  // Random weights: approximately normal with this standard deviation, or (uniform) in [lo, hi).
  bool uniform = false;
  double p0 = 0.02, p1 = 0.0;     // normal: p0 = standard deviation; uniform: p0 = lo, p1 = hi
};

struct HostArray {
  std::vector<int32_t> data;
  std::vector<int64_t> shape;
};

// What the host knows of a step before anything is uploaded.
struct HostStep {
  std::vector<int> q_lens, starts, k_lens, state_slots;
  int k_len_bound = 0;            // no k_len is larger
  bool frozen = false;            // the step is recorded for replay: launches must cover k_len_bound keys
  std::map<std::string, std::shared_ptr<void>> memo;   // parts keep what they derive once per step here
};

struct GroupTables {
  Tensor slots;                   // [T] cache slot of every token, -1: store nothing
  Tensor block_table;             // [S, width]
  int window = 0;
};

struct StepContext {
  Kernels* kernels = nullptr;
  int num_tokens = 0, num_seqs = 0;
  Tensor positions, cu_q, k_len, state_slots;
  std::vector<GroupTables> groups;
  HostStep* host = nullptr;
  std::map<std::string, Tensor> inputs;              // the arrays parts asked for, on the GPU
  std::function<Tensor(int64_t)> workspace;           // float32 scratch of at least that many elements
};

// What a mixer keeps between steps.
struct CacheNeed {
  enum Kind { None, Pages, State } kind = None;
  int num_kv_heads = 0, head_dim = 0, window = 0;    // Pages
  std::vector<int64_t> state_shape;                  // State: per request
  DType state_dtype = DType::F32;
};

struct CacheEntry {
  CacheNeed::Kind kind = CacheNeed::None;
  Tensor k, v;                    // [pages, kv heads, page, d] and [pages, kv heads, d, page]
  int group = 0, page_size = 0;
  bool writable = true;           // false: the keys and values are an earlier execution's
  Tensor state;                   // [slots, ...]
};

class Part {
 public:
  explicit Part(Kernels& k) : kernels(k) {}
  virtual ~Part() = default;
  virtual std::vector<ParamDecl> params() const { return {}; }
  virtual std::vector<std::pair<std::string, Part*>> children() { return {}; }
  virtual void load(std::map<std::string, Tensor>& tensors) { (void)tensors; }
  // Parts that need arrays of their own in every step name them with one key per kind of array set; the
  // step function asks one part per key and uploads the arrays with the step's other numbers.
  virtual const char* step_inputs_key() const { return nullptr; }
  virtual void step_inputs(HostStep& step, std::vector<std::pair<std::string, HostArray>>& out) { (void)step; (void)out; }
  virtual int64_t workspace_floats(HostStep& step) { (void)step; return 0; }
  // false: the part's launches depend on the step's host numbers (HostStep) and not only on the arrays on the
  // GPU, so a recorded step would repeat one step's numbers; a model with such a part is never recorded.
  virtual bool replayable() const { return true; }

 protected:
  Kernels& kernels;
};

class Embedding : public Part {
 public:
  using Part::Part;
  virtual Tensor forward(const Tensor& ids) = 0;
};

class Norm : public Part {
 public:
  using Part::Part;
  virtual Tensor forward(const Tensor& x) = 0;
  // residual += x in place (the sum in 32-bit, stored rounded); returns the norm of the unrounded sum.
  virtual Tensor forward_add(const Tensor& x, Tensor& residual) = 0;
  // A norm that is y = x * rsqrt(mean(x^2) + eps) * w says so; a mixer may then run it inside a launch of its own.
  virtual const Tensor* row_scale_weight() const { return nullptr; }
  virtual float eps() const { return 0.f; }
};

class PositionEncoding : public Part {
 public:
  using Part::Part;
  // A rotation by tabulated angles gives its tables [positions, half]; a mixer may then rotate inside a launch of its own.
  virtual const Tensor* cos_table() { return nullptr; }
  virtual const Tensor* sin_table() { return nullptr; }
  // Encodes positions [T] into q [T, heads, d] and k [T, kv heads, d]; k may have no memory (only q is wanted).
  // The default rotates by the tables above; a kind without tables brings its own.
  virtual std::pair<Tensor, Tensor> apply(const Tensor& q, const Tensor& k, const Tensor& positions);
};

class Mixer : public Part {
 public:
  using Part::Part;
  virtual CacheNeed cache_need() const = 0;
  virtual Tensor forward(const Tensor& x, StepContext& ctx, CacheEntry& cache) = 0;
};

class FeedForward : public Part {
 public:
  using Part::Part;
  virtual Tensor forward(const Tensor& x, StepContext& ctx) = 0;
};

class Head : public Part {
 public:
  using Part::Part;
  virtual Tensor forward(const Tensor& x) = 0;
};

class Block : public Part {
 public:
  using Part::Part;
  virtual Mixer& mixer() = 0;
  // (hidden, residual) -> (hidden, residual); `residual` has no memory before the first layer.
  virtual std::pair<Tensor, Tensor> forward(const Tensor& hidden, Tensor residual, StepContext& ctx, CacheEntry& cache) = 0;
};

using PartFactory = std::function<std::unique_ptr<Part>(const PartSpec&, Kernels&)>;
using BlockFactory = std::function<std::unique_ptr<Block>(Kernels&, std::unique_ptr<Mixer>, std::unique_ptr<FeedForward>,
                                                          std::map<std::string, std::unique_ptr<Norm>>)>;
// category: "embedding", "norm", "position", "mixer", "feed_forward", "head".
void register_part(const std::string& category, const std::string& kind, PartFactory make);
void register_block(const std::string& kind, BlockFactory make);
std::unique_ptr<Part> build_any_part(const std::string& category, const PartSpec& spec, Kernels& k);
std::unique_ptr<Block> build_block(const LayerSpec& spec, Kernels& k);

template <class T>
std::unique_ptr<T> build_part(const std::string& category, const PartSpec& spec, Kernels& k) {
  std::unique_ptr<Part> p = build_any_part(category, spec, k);
  T* t = dynamic_cast<T*>(p.get());
  if (!t) throw ConfigError("part '" + spec.kind + "' is registered as '" + category + "' but has another interface");
  p.release();
  return std::unique_ptr<T>(t);
}

void register_standard_parts();   // the kinds the Qwen3 dense decoder is made of
bool part_registered(const std::string& category, const std::string& kind);
bool block_registered(const std::string& kind);
// Why this registry cannot build the model, or "" if it can: the first part or block kind that is missing.
std::string missing_part(const ModelSpec& spec);

// Loads a shared library and calls its `extern "C" void vosti_plugin_register(void)`, in which it registers
// part kinds (register_part, register_block) and architectures (register_architecture).  A path is loaded once.
void load_plugin(const std::string& path);

}  // namespace vosti
