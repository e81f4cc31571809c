#include "parts.h"

#include "../host/rules.h"

#include <dlfcn.h>

#include <cmath>
#include <mutex>

namespace vosti {

// --------------------------------------------------------------------------------------- registry
namespace {
std::map<std::pair<std::string, std::string>, PartFactory>& part_registry() {
  static std::map<std::pair<std::string, std::string>, PartFactory> r;
  return r;
}
std::map<std::string, BlockFactory>& block_registry() {
  static std::map<std::string, BlockFactory> r;
  return r;
}
}  // namespace

void register_part(const std::string& category, const std::string& kind, PartFactory make) {
  part_registry()[{category, kind}] = std::move(make);
}
void register_block(const std::string& kind, BlockFactory make) { block_registry()[kind] = std::move(make); }
bool part_registered(const std::string& category, const std::string& kind) { return part_registry().count({category, kind}) > 0; }
bool block_registered(const std::string& kind) { return block_registry().count(kind) > 0; }

namespace {
std::string missing_in(const std::string& category, const PartSpec& p) {
  if (!part_registered(category, p.kind)) return category + " part '" + p.kind + "'";
  // Parts below a part: the name says the category ("q_norm", "k_norm": norms; "position").
  for (const auto& c : p.parts) {
    const std::string below = c.first == "position" ? "position" : (c.first.size() >= 4 && c.first.compare(c.first.size() - 4, 4, "norm") == 0 ? "norm" : "");
    if (below.empty()) continue;
    const std::string m = missing_in(below, *c.second);
    if (!m.empty()) return m;
  }
  return "";
}
}  // namespace

std::string missing_part(const ModelSpec& spec) {
  std::string m = missing_in("embedding", *spec.embedding);
  if (m.empty()) m = missing_in("norm", *spec.final_norm);
  if (m.empty()) m = missing_in("head", *spec.head);
  for (const LayerSpec& l : spec.layers) {
    if (!m.empty()) break;
    if (!block_registered(l.block)) m = "block arrangement '" + l.block + "'";
    if (m.empty()) m = missing_in("mixer", *l.mixer);
    if (m.empty()) m = missing_in("feed_forward", *l.feed_forward);
    for (const auto& n : l.norms)
      if (m.empty()) m = missing_in("norm", *n.second);
  }
  return m;
}

void load_plugin(const std::string& path) {
  static std::mutex mutex;
  static std::map<std::string, void*> loaded;
  std::lock_guard<std::mutex> lock(mutex);
  if (loaded.count(path)) return;
  void* h = dlopen(path.c_str(), RTLD_NOW | RTLD_GLOBAL);
  if (!h) throw EngineError("cannot load the plugin " + path + ": " + dlerror());
  auto fn = reinterpret_cast<void (*)()>(dlsym(h, "vosti_plugin_register"));
  if (!fn) throw EngineError("the plugin " + path + " has no vosti_plugin_register()");
  register_standard_parts();
  register_builtin_architectures();
  fn();
  loaded[path] = h;
}

std::pair<Tensor, Tensor> PositionEncoding::apply(const Tensor& q, const Tensor& k, const Tensor& positions) {
  const Tensor *cos = cos_table(), *sin = sin_table();
  if (!cos || !sin) throw EngineError("a position encoding needs tables of angles or an apply() of its own");
  auto rotate = [&](const Tensor& x) {
    if (x.shape.size() != 3) throw EngineError("position encoding of " + x.describe() + ", expected [tokens, heads, head size]");
    const int64_t T = x.dim(0), n = x.dim(1), d = x.dim(2);
    return kernels.qkv_post(x.view({T, n * d}), (int)n, 0, (int)d, nullptr, nullptr, 0, nullptr, nullptr, 0.f, cos, sin, &positions, nullptr);
  };
  return {rotate(q), k.data ? rotate(k) : Tensor()};
}

std::unique_ptr<Part> build_any_part(const std::string& category, const PartSpec& spec, Kernels& k) {
  auto it = part_registry().find({category, spec.kind});
  if (it == part_registry().end()) throw ConfigError("no " + category + " part of kind '" + spec.kind + "' in the native engine");
  return it->second(spec, k);
}

std::unique_ptr<Block> build_block(const LayerSpec& spec, Kernels& k) {
  auto it = block_registry().find(spec.block);
  if (it == block_registry().end()) throw ConfigError("no block arrangement of kind '" + spec.block + "' in the native engine");
  std::map<std::string, std::unique_ptr<Norm>> norms;
  for (const auto& n : spec.norms) norms[n.first] = build_part<Norm>("norm", *n.second, k);
  return it->second(k, build_part<Mixer>("mixer", *spec.mixer, k), build_part<FeedForward>("feed_forward", *spec.feed_forward, k),
                    std::move(norms));
}

namespace {

Tensor need(std::map<std::string, Tensor>& tensors, const std::string& name) {
  auto it = tensors.find(name);
  if (it == tensors.end()) throw EngineError("a part was not given its tensor '" + name + "'");
  return it->second;
}

// Rows of several weights one under the other in one buffer, so that one launch projects them all.
Tensor stack_rows(const std::vector<Tensor>& pieces) {
  int64_t rows = 0;
  for (const Tensor& p : pieces) {
    if (p.shape.size() != 2 || p.dim(1) != pieces[0].dim(1) || p.dtype != pieces[0].dtype)
      throw EngineError("weights that are stacked must have one width and one type");
    rows += p.dim(0);
  }
  Tensor out;
  out.dtype = pieces[0].dtype;
  out.shape = {rows, pieces[0].dim(1)};
  out.owner = std::make_shared<DeviceBuffer>(out.bytes());
  out.data = out.owner->data();
  size_t at = 0;
  for (const Tensor& p : pieces) {
    hip_check(hipMemcpy(static_cast<char*>(out.data) + at, p.data, p.bytes(), hipMemcpyDeviceToDevice), "stacking weights");
    at += p.bytes();
  }
  return out;
}

// h[t] = E[ids[t]], a row copy without scale (src/exec/dense_swiglu_model.rs:271-273).
class TokenEmbedding : public Embedding {
 public:
  TokenEmbedding(const PartSpec& s, Kernels& k) : Embedding(k), vocab_(s.integer("vocab_size")), hidden_(s.integer("hidden_size")) {}
  std::vector<ParamDecl> params() const override { return {{"weight", {vocab_, hidden_}}}; }
  void load(std::map<std::string, Tensor>& t) override { weight_ = need(t, "weight"); }
  Tensor forward(const Tensor& ids) override { return kernels.embedding(weight_, ids); }

 private:
  int64_t vocab_, hidden_;
  Tensor weight_;
};

// y = (x * rsqrt(mean(x^2) + eps)) * w in 32-bit (kernels/triton_kernels/rmsnorm.py:63-93); with a residual
// the norm sees the unrounded sum (kernels/triton_kernels/rmsnorm_residual.py:73-125).
class RMSNorm : public Norm {
 public:
  RMSNorm(const PartSpec& s, Kernels& k) : Norm(k), size_(s.integer("size")), eps_((float)s.number("eps")) {}
  std::vector<ParamDecl> params() const override { return {{"weight", {size_}, true, true, 0.9, 1.1}}; }
  void load(std::map<std::string, Tensor>& t) override { weight_ = need(t, "weight"); }
  Tensor forward(const Tensor& x) override { return kernels.rmsnorm(x, weight_, eps_); }
  Tensor forward_add(const Tensor& x, Tensor& residual) override { return kernels.add_rmsnorm(x, residual, weight_, eps_); }
  const Tensor* row_scale_weight() const override { return &weight_; }
  float eps() const override { return eps_; }

 private:
  int64_t size_;
  float eps_;
  Tensor weight_;
};

// Half-rotation rotary encoding with tables (python/vosti_kernels/rotary.py:80-90 for the frequencies,
// :137-160 for the tables, kernels/triton_kernels/rope.py:78-123 for the rotation).  inv_freq[j] =
// 1 / theta^(2j / rotary_dim) is computed once on the host in 32-bit (rotary_inverse_frequencies, the one
// routine every host of these kernels uses); the angles, cosines and sines of every position are computed on
// the GPU in 32-bit and stored as elements.
class Rotary : public PositionEncoding {
 public:
  Rotary(const PartSpec& s, Kernels& k)
      : PositionEncoding(k), head_dim_(s.integer("head_dim")), rotary_dim_(s.integer("rotary_dim")), theta_(s.number("theta")),
        max_positions_(s.integer("max_positions")) {
    if (rotary_dim_ % 2 || rotary_dim_ <= 0 || rotary_dim_ > head_dim_)
      throw ConfigError("rotary width " + std::to_string(rotary_dim_) + " must be even and at most the head size " + std::to_string(head_dim_));
  }
  const Tensor* cos_table() override { return &ensure().first; }
  const Tensor* sin_table() override { return &ensure().second; }

 private:
  using Tables = std::pair<Tensor, Tensor>;
  const Tables& ensure() {
    if (tables_) return *tables_;
    // Layers with the same geometry share one pair of tables.
    static std::map<std::tuple<std::string, int64_t, double, int64_t>, std::shared_ptr<Tables>> shared;
    auto key = std::make_tuple(kernels.name(), rotary_dim_, theta_, max_positions_);
    auto it = shared.find(key);
    if (it == shared.end()) {
      const int64_t half = rotary_dim_ / 2;
      std::vector<float> inv(half);
      rotary_inverse_frequencies(theta_, (int)rotary_dim_, inv.data());
      DeviceBuffer inv_dev(half * sizeof(float));
      hip_check(hipMemcpy(inv_dev.data(), inv.data(), half * sizeof(float), hipMemcpyHostToDevice), "rotary frequencies");
      Tensor inv_t;
      inv_t.data = inv_dev.data();
      inv_t.dtype = DType::F32;
      inv_t.shape = {half};
      auto tables = std::make_shared<Tables>();
      for (Tensor* t : {&tables->first, &tables->second}) {
        t->dtype = kernels.dtype();
        t->shape = {max_positions_, half};
        t->owner = std::make_shared<DeviceBuffer>(t->bytes());
        t->data = t->owner->data();
      }
      kernels.rope_tables(tables->first, tables->second, inv_t);
      hip_check(hipStreamSynchronize(kernels.stream), "rotary tables");
      it = shared.emplace(key, tables).first;
    }
    tables_ = it->second;
    return *tables_;
  }
  int64_t head_dim_, rotary_dim_;
  double theta_;
  int64_t max_positions_;
  std::shared_ptr<Tables> tables_;
};

// The attention kernels work on items: a single decoded token, or up to item_rows() consecutive rows of a
// sequence that brings several tokens.  The item lists are the same for every attention layer of a step.
struct AttentionItems {
  HostArray prefill, decode;
  int decode_bound = 0, nseg = 0;
};

// Causal grouped-query attention over the paged cache (src/exec/dense_swiglu_decoder.rs:171-367): QKV
// projection without bias, per-head norm of q and k, rotary encoding, store of k and v, attention, output
// projection.  window > 0 limits a query to that many last keys.  q_norm, k_norm and position are parts of
// their own; when they are weighted row scales and a rotation by tables the three steps between the projections
// run as one launch.
class Attention : public Mixer {
 public:
  Attention(const PartSpec& s, Kernels& k)
      : Mixer(k), hidden_(s.integer("hidden_size")), nq_((int)s.integer("num_heads")), nkv_((int)s.integer("num_kv_heads")),
        d_((int)s.integer("head_dim")), scale_((float)s.number("scale")), window_((int)s.integer("window", 0)) {
    if (nq_ % nkv_) throw ConfigError(std::to_string(nq_) + " heads are not a multiple of " + std::to_string(nkv_) + " kv heads");
    if (d_ % 16 || d_ < 16 || d_ > 256)
      throw ConfigError("head size " + std::to_string(d_) + ": the attention kernels take multiples of 16 from 16 to 256");
    if (const PartSpec* p = s.part("q_norm")) q_norm_ = build_part<Norm>("norm", *p, k);
    if (const PartSpec* p = s.part("k_norm")) k_norm_ = build_part<Norm>("norm", *p, k);
    if (const PartSpec* p = s.part("position")) position_ = build_part<PositionEncoding>("position", *p, k);
  }
  std::vector<ParamDecl> params() const override {
    return {{"q_proj.weight", {(int64_t)nq_ * d_, hidden_}}, {"k_proj.weight", {(int64_t)nkv_ * d_, hidden_}},
            {"v_proj.weight", {(int64_t)nkv_ * d_, hidden_}}, {"o_proj.weight", {hidden_, (int64_t)nq_ * d_}}};
  }
  std::vector<std::pair<std::string, Part*>> children() override {
    std::vector<std::pair<std::string, Part*>> c;
    if (q_norm_) c.emplace_back("q_norm", q_norm_.get());
    if (k_norm_) c.emplace_back("k_norm", k_norm_.get());
    if (position_) c.emplace_back("position", position_.get());
    return c;
  }
  void load(std::map<std::string, Tensor>& t) override {
    // One launch projects q, k and v (kernels/triton_kernels/qkv_matmul.py:108-211); rows of the fused
    // weight are q's, then k's, then v's.
    w_qkv_ = stack_rows({need(t, "q_proj.weight"), need(t, "k_proj.weight"), need(t, "v_proj.weight")});
    w_o_ = need(t, "o_proj.weight");
  }
  // Head norms, rotation and cache store run as one launch when the norms are weighted row scales with one eps
  // and the position encoding is a rotation by tables; any other kind runs through its own methods, step by step.
  // Asked when the sub-parts have their tensors (a norm's weight, a rotation's tables).
  bool fused() {
    for (Norm* n : {q_norm_.get(), k_norm_.get()})
      if (n && !n->row_scale_weight()) return false;
    if (q_norm_ && k_norm_ && q_norm_->eps() != k_norm_->eps()) return false;
    return !position_ || position_->cos_table() != nullptr;
  }
  CacheNeed cache_need() const override {
    CacheNeed n;
    n.kind = CacheNeed::Pages;
    n.num_kv_heads = nkv_;
    n.head_dim = d_;
    n.window = window_;
    return n;
  }
  const char* step_inputs_key() const override { return "attention.items"; }

  AttentionItems& items(HostStep& step) {
    auto it = step.memo.find("attention.items");
    if (it != step.memo.end()) return *static_cast<AttentionItems*>(it->second.get());
    auto m = std::make_shared<AttentionItems>();
    const int rows = kernels.item_rows();
    int decode_keys = 0;
    for (size_t s = 0; s < step.q_lens.size(); ++s) {
      if (step.q_lens[s] == 1) {
        m->decode.data.push_back((int32_t)s);
        m->decode.data.push_back(0);
        decode_keys = std::max(decode_keys, step.k_lens[s]);
      } else {
        for (int off = 0; off < step.q_lens[s]; off += rows) {
          m->prefill.data.push_back((int32_t)s);
          m->prefill.data.push_back(off);
        }
      }
    }
    m->prefill.shape = {(int64_t)m->prefill.data.size() / 2, 2};
    m->decode.shape = {(int64_t)m->decode.data.size() / 2, 2};
    // Recorded launches must cover every length that the tables can hold.
    m->decode_bound = step.frozen ? step.k_len_bound : decode_keys;
    m->nseg = (m->decode_bound + kernels.segment_keys() - 1) / kernels.segment_keys();
    step.memo["attention.items"] = m;
    return *m;
  }
  void step_inputs(HostStep& step, std::vector<std::pair<std::string, HostArray>>& out) override {
    AttentionItems& m = items(step);
    out.emplace_back("attention.prefill_items", m.prefill);
    out.emplace_back("attention.decode_items", m.decode);
  }
  // Workspace with which the two projections of T rows take their faster route, where there is one.
  int64_t gemm_floats(int64_t T) const {
    return std::max(kernels.gemm_workspace_floats(T, (int64_t)(nq_ + 2 * nkv_) * d_, hidden_),
                    kernels.gemm_workspace_floats(T, hidden_, (int64_t)nq_ * d_));
  }
  int64_t workspace_floats(HostStep& step) override {
    AttentionItems& m = items(step);
    int64_t T = 0;
    for (int q : step.q_lens) T += q;
    int64_t need = gemm_floats(T);
    if (m.decode.shape[0]) need = std::max(need, kernels.attn_scratch_floats((int)m.decode.shape[0], nq_, d_, m.nseg));
    return need;
  }

  Tensor forward(const Tensor& x, StepContext& ctx, CacheEntry& cache) override {
    if (cache.kind != CacheNeed::Pages) throw EngineError("attention was handed a cache entry without pages");
    Kernels& k = kernels;
    const int64_t T = x.dim(0);
    GroupTables& tables = ctx.groups.at(cache.group);
    // Without a cache of its own the keys and values are an earlier execution's: only q is projected.
    // The projections, the attention of decoded tokens and the next projection use the step's workspace one
    // after the other.
    const int64_t gf = gemm_floats(T);
    Tensor ws_t;
    if (gf) ws_t = ctx.workspace(gf);
    const Tensor* ws = gf ? &ws_t : nullptr;
    const Tensor qkv = k.gemm(x, cache.writable ? w_qkv_ : w_qkv_.rows(0, (int64_t)nq_ * d_), ws);
    Tensor q;
    if (fused()) {
      const Norm* en = q_norm_ ? q_norm_.get() : k_norm_.get();
      q = k.qkv_post(qkv, nq_, cache.writable ? nkv_ : 0, d_, &cache.k, &cache.v, cache.page_size,
                     q_norm_ ? q_norm_->row_scale_weight() : nullptr, k_norm_ ? k_norm_->row_scale_weight() : nullptr,
                     en ? en->eps() : 0.f, position_ ? position_->cos_table() : nullptr,
                     position_ ? position_->sin_table() : nullptr, &ctx.positions, &tables.slots);
    } else {
      q = unfused(qkv, ctx, cache, tables);
    }
    Tensor out = k.empty(q.shape);
    AttentionItems& m = items(*ctx.host);
    const Tensor& prefill_items = ctx.inputs.at("attention.prefill_items");
    const Tensor& decode_items = ctx.inputs.at("attention.decode_items");
    if (prefill_items.dim(0))
      k.paged_attention(out, q, cache.k, cache.v, tables.block_table, ctx.cu_q, ctx.k_len, prefill_items, 0, scale_, window_,
                        ctx.host->k_len_bound, 0, nullptr);
    if (decode_items.dim(0)) {
      const Tensor scratch = ctx.workspace(k.attn_scratch_floats((int)decode_items.dim(0), nq_, d_, m.nseg));
      k.paged_attention(out, q, cache.k, cache.v, tables.block_table, ctx.cu_q, ctx.k_len, decode_items, 1, scale_, window_,
                        m.decode_bound, m.nseg, &scratch);
    }
    return k.gemm(out.view({T, (int64_t)nq_ * d_}), w_o_, ws);
  }

 private:
  // Norm, position encoding and store as separate steps, each sub-part through its own methods.
  Tensor unfused(const Tensor& qkv, StepContext& ctx, CacheEntry& cache, GroupTables& tables) {
    Kernels& k = kernels;
    const int64_t T = qkv.dim(0), qw = (int64_t)nq_ * d_, kw = (int64_t)nkv_ * d_;
    Tensor q = k.columns(qkv, 0, qw).view({T, nq_, d_});
    if (q_norm_) q = q_norm_->forward(q);
    if (!cache.writable) {
      if (position_) q = position_->apply(q, Tensor(), ctx.positions).first;
      return q;
    }
    Tensor kk = k.columns(qkv, qw, kw).view({T, nkv_, d_});
    if (k_norm_) kk = k_norm_->forward(kk);
    if (position_) std::tie(q, kk) = position_->apply(q, kk, ctx.positions);
    Tensor kv = k.empty({T, 2 * kw});
    k.copy_columns(kv, 0, kk.view({T, kw}), 0, kw);
    k.copy_columns(kv, kw, qkv, qw + kw, kw);
    k.qkv_post(kv, 0, nkv_, d_, &cache.k, &cache.v, cache.page_size, nullptr, nullptr, 0.f, nullptr, nullptr, nullptr, &tables.slots);
    return q;
  }

  int64_t hidden_;
  int nq_, nkv_, d_;
  float scale_;
  int window_;
  std::unique_ptr<Norm> q_norm_, k_norm_;
  std::unique_ptr<PositionEncoding> position_;
  Tensor w_qkv_, w_o_;
};

// down(silu(gate(x)) * up(x)) without biases (src/exec/dense_swiglu_decoder.rs:396-438); gate and up are one
// projection whose output is rounded before the activation
// (python/vosti_kernels/model_families/qwen3/loader.py:55-58, kernels/triton_kernels/silu_mul.py:64-87).
class SwiGLU : public FeedForward {
 public:
  SwiGLU(const PartSpec& s, Kernels& k) : FeedForward(k), hidden_(s.integer("hidden_size")), inter_(s.integer("intermediate_size")) {}
  std::vector<ParamDecl> params() const override {
    return {{"gate_proj.weight", {inter_, hidden_}}, {"up_proj.weight", {inter_, hidden_}}, {"down_proj.weight", {hidden_, inter_}}};
  }
  void load(std::map<std::string, Tensor>& t) override {
    w_gate_up_ = stack_rows({need(t, "gate_proj.weight"), need(t, "up_proj.weight")});
    w_down_ = need(t, "down_proj.weight");
  }
  int64_t gemm_floats(int64_t T) const {
    return std::max(kernels.gemm_workspace_floats(T, 2 * inter_, hidden_, true), kernels.gemm_workspace_floats(T, hidden_, inter_));
  }
  int64_t workspace_floats(HostStep& step) override {
    int64_t T = 0;
    for (int q : step.q_lens) T += q;
    return gemm_floats(T);
  }
  Tensor forward(const Tensor& x, StepContext& ctx) override {
    const int64_t n = gemm_floats(x.dim(0));
    Tensor ws;
    if (n) ws = ctx.workspace(n);
    return kernels.gemm(kernels.gemm_swiglu(x, w_gate_up_, n ? &ws : nullptr), w_down_, n ? &ws : nullptr);
  }

 private:
  int64_t hidden_, inter_;
  Tensor w_gate_up_, w_down_;
};

// x += mixer(norm(x)); x += ffn(norm(x)), carried as (hidden, residual) so that each add runs inside the
// next norm (src/exec/dense_swiglu_decoder.rs:556-615 first layer, :740-813 others).
class PreNormBlock : public Block {
 public:
  PreNormBlock(Kernels& k, std::unique_ptr<Mixer> mixer, std::unique_ptr<FeedForward> ffn, std::map<std::string, std::unique_ptr<Norm>> norms)
      : Block(k), mixer_(std::move(mixer)), ffn_(std::move(ffn)), norms_(std::move(norms)) {
    for (const char* n : {"input", "post_mixer"})
      if (!norms_.count(n)) throw ConfigError(std::string("a prenorm block needs the norms 'input' and 'post_mixer'; missing: ") + n);
  }
  std::vector<std::pair<std::string, Part*>> children() override {
    std::vector<std::pair<std::string, Part*>> c = {{"mixer", mixer_.get()}, {"feed_forward", ffn_.get()}};
    for (auto& n : norms_) c.emplace_back("norms." + n.first, n.second.get());
    return c;
  }
  Mixer& mixer() override { return *mixer_; }
  std::pair<Tensor, Tensor> forward(const Tensor& hidden, Tensor residual, StepContext& ctx, CacheEntry& cache) override {
    Tensor normed;
    if (residual.data == nullptr) {
      residual = hidden;
      normed = norms_["input"]->forward(hidden);
    } else {
      normed = norms_["input"]->forward_add(hidden, residual);
    }
    const Tensor mixed = mixer_->forward(normed, ctx, cache);
    normed = norms_["post_mixer"]->forward_add(mixed, residual);
    return {ffn_->forward(normed, ctx), residual};
  }

 private:
  std::unique_ptr<Mixer> mixer_;
  std::unique_ptr<FeedForward> ffn_;
  std::map<std::string, std::unique_ptr<Norm>> norms_;
};

// logits = x W^T without bias (src/exec/dense_swiglu_model.rs:976-984).  A head tied to the embedding is this
// same part: the architecture gives its weight the embedding table's tensor name, and the model hands both
// parts the one tensor (python/vosti_kernels/model_families/qwen3/physical.py:131-134).
class LinearHead : public Head {
 public:
  LinearHead(const PartSpec& s, Kernels& k) : Head(k), vocab_(s.integer("vocab_size")), hidden_(s.integer("hidden_size")) {}
  std::vector<ParamDecl> params() const override { return {{"weight", {vocab_, hidden_}}}; }
  void load(std::map<std::string, Tensor>& t) override { weight_ = need(t, "weight"); }
  Tensor forward(const Tensor& x) override { return kernels.gemm(x, weight_); }

 private:
  int64_t vocab_, hidden_;
  Tensor weight_;
};

template <class T>
PartFactory factory() {
  return [](const PartSpec& s, Kernels& k) { return std::unique_ptr<Part>(new T(s, k)); };
}

}  // namespace

void register_standard_parts() {
  static std::once_flag once;
  std::call_once(once, [] {
    register_part("embedding", "token_embedding", factory<TokenEmbedding>());
    register_part("norm", "rmsnorm", factory<RMSNorm>());
    register_part("position", "rotary", factory<Rotary>());
    register_part("mixer", "attention", factory<Attention>());
    register_part("feed_forward", "swiglu", factory<SwiGLU>());
    register_part("head", "linear_head", factory<LinearHead>());
    register_block("prenorm", [](Kernels& k, std::unique_ptr<Mixer> m, std::unique_ptr<FeedForward> f,
                                 std::map<std::string, std::unique_ptr<Norm>> n) {
      return std::unique_ptr<Block>(new PreNormBlock(k, std::move(m), std::move(f), std::move(n)));
    });
  });
}

}  // namespace vosti
