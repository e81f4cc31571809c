// A plugin of the native engine, for tests: a position encoding, a mixer with state of its own and two
// architectures that the engine's own files know nothing of.  Compiled by the test with the host compiler against
// csrc/engine/parts.h and loaded with load_plugin(); they are toys, never models of anyone's.
//
// "toy_scaled_half_rotary": a half-rotation of the first half of each head only, at positions scaled down by
// `factor` (angle = inv_freq[j] * p / factor, inv_freq over the rotated width).  It offers no tables to the
// mixer, so the attention part cannot run it inside its fused launch and has to call apply().
//
// "ToyScaledRopeForCausalLM": the Qwen3 decoder with that encoding in every layer; config.json has the Qwen3
// keys and "toy_rope_factor".
//
// "toy_carry": a mixer that keeps one vector per request in a state slot.  z_t = W x_t;  u_t = s_{t-1} + z_t
// (s before a request's first token is zero);  y_t = u_t * rsqrt(mean(u_t^2) + eps) * gain;  s_t = u_t rounded to
// the model's type.  It walks the step's host numbers token by token, so it says that it cannot be replayed.
//
// "ToyNativeHybridForCausalLM": three layers (attention over all keys with head norms and the standard rotation;
// toy_carry; attention over a window of keys with the toy encoding and no head norms, so two cache groups), each
// with a SwiGLU feed-forward, run in the order 0, 1, 2, 0, 2, where the second execution of layer 0 has a cache of
// its own and the second execution of layer 2 reads the keys and values that its first execution stored.
#include <cmath>
#include <cstring>

#include "../vosti_amd/csrc/engine/parts.h"
#include "../vosti_amd/csrc/host/qwen3.h"
#include "../vosti_amd/csrc/host/rules.h"

using namespace vosti;

namespace {

class ScaledHalfRotary : public PositionEncoding {
 public:
  ScaledHalfRotary(const PartSpec& s, Kernels& k)
      : PositionEncoding(k), rotary_dim_(s.integer("rotary_dim")), theta_(s.number("theta")), factor_(s.number("factor")),
        max_positions_(s.integer("max_positions")) {}

  std::pair<Tensor, Tensor> apply(const Tensor& q, const Tensor& k, const Tensor& positions) override {
    ensure();
    auto rotate = [&](const Tensor& x) {
      const int64_t T = x.dim(0), n = x.dim(1), d = x.dim(2);
      return kernels.qkv_post(x.view({T, n * d}), (int)n, 0, (int)d, nullptr, nullptr, 0, nullptr, nullptr, 0.f, &cos_, &sin_, &positions, nullptr);
    };
    return {rotate(q), k.data ? rotate(k) : Tensor()};
  }

 private:
  void ensure() {
    if (cos_.data) return;
    const int64_t half = rotary_dim_ / 2;
    std::vector<float> inv((size_t)half);
    rotary_inverse_frequencies(theta_, (int)rotary_dim_, inv.data());
    for (float& f : inv) f = f / (float)factor_;
    DeviceBuffer inv_dev((size_t)half * sizeof(float));
    hip_check(hipMemcpy(inv_dev.data(), inv.data(), (size_t)half * sizeof(float), hipMemcpyHostToDevice), "toy frequencies");
    Tensor inv_t;
    inv_t.data = inv_dev.data();
    inv_t.dtype = DType::F32;
    inv_t.shape = {half};
    for (Tensor* t : {&cos_, &sin_}) {
      t->dtype = kernels.dtype();
      t->shape = {max_positions_, half};
      t->owner = std::make_shared<DeviceBuffer>(t->bytes());
      t->data = t->owner->data();
    }
    kernels.rope_tables(cos_, sin_, inv_t);
    hip_check(hipStreamSynchronize(kernels.stream), "toy tables");
  }
  int64_t rotary_dim_;
  double theta_, factor_;
  int64_t max_positions_;
  Tensor cos_, sin_;
};

ModelSpec toy_scaled_rope(const Json& raw) {
  Json as_qwen3 = raw;
  for (auto& m : as_qwen3.members)
    if (m.first == "model_type") m.second.text = "qwen3";
  const Json* factor = raw.get("toy_rope_factor");
  if (!factor || factor->kind != Json::Number || factor->number <= 0) throw ConfigError("config.json: 'toy_rope_factor' must be a positive number");
  const Qwen3Config c = qwen3_config(as_qwen3);
  if (c.head_dim % 4) throw ConfigError("config.json: 'head_dim' must be a multiple of 4 for the toy encoding");
  ModelSpec spec = qwen3_model_spec(c);
  spec.architecture = "ToyScaledRopeForCausalLM";
  auto position = std::make_shared<PartSpec>();
  position->kind = "toy_scaled_half_rotary";
  position->numbers = {{"rotary_dim", (double)(c.head_dim / 2)}, {"theta", c.rope_theta}, {"factor", factor->number},
                       {"max_positions", (double)c.max_position_embeddings}};
  for (LayerSpec& l : spec.layers) {
    auto mixer = std::make_shared<PartSpec>(*l.mixer);
    mixer->parts["position"] = position;
    l.mixer = mixer;
  }
  return spec;
}

class Carry : public Mixer {
 public:
  Carry(const PartSpec& s, Kernels& k) : Mixer(k), hidden_(s.integer("hidden_size")), eps_((float)s.number("eps")) {}
  std::vector<ParamDecl> params() const override {
    ParamDecl gain{"gain", {hidden_}};
    gain.uniform = true;
    gain.p0 = 0.5;
    gain.p1 = 1.5;
    return {{"in_proj.weight", {hidden_, hidden_}}, gain};
  }
  void load(std::map<std::string, Tensor>& t) override {
    w_ = t.at("in_proj.weight");
    gain_ = t.at("gain");
  }
  CacheNeed cache_need() const override {
    CacheNeed n;
    n.kind = CacheNeed::State;
    n.state_shape = {hidden_};
    n.state_dtype = kernels.dtype();
    return n;
  }
  bool replayable() const override { return false; }

  Tensor forward(const Tensor& x, StepContext& ctx, CacheEntry& cache) override {
    if (cache.kind != CacheNeed::State) throw EngineError("toy_carry was handed a cache entry without state");
    const Tensor z = kernels.gemm(x, w_);
    Tensor y = kernels.empty(x.shape);
    const size_t row_bytes = (size_t)hidden_ * dtype_bytes(kernels.dtype());
    int64_t row = 0;
    for (size_t s = 0; s < ctx.host->q_lens.size(); ++s) {
      Tensor state = cache.state.rows(ctx.host->state_slots[s], 1);
      if (ctx.host->starts[s] == 0) hip_check(hipMemsetAsync(state.data, 0, row_bytes, kernels.stream), "toy_carry: clearing a state");
      for (int t = 0; t < ctx.host->q_lens[s]; ++t, ++row) {
        const Tensor out = kernels.add_rmsnorm(z.rows(row, 1), state, gain_, eps_);
        hip_check(hipMemcpyAsync(static_cast<char*>(y.data) + (size_t)row * row_bytes, out.data, row_bytes, hipMemcpyDeviceToDevice, kernels.stream),
                  "toy_carry: copying a row");
      }
    }
    return y;
  }

 private:
  int64_t hidden_;
  float eps_;
  Tensor w_, gain_;
};

PartSpecPtr make_part(std::string kind, std::map<std::string, double> numbers, std::map<std::string, PartSpecPtr> parts = {}) {
  auto p = std::make_shared<PartSpec>();
  p->kind = std::move(kind);
  p->numbers = std::move(numbers);
  p->parts = std::move(parts);
  return p;
}

ModelSpec toy_native_hybrid(const Json& raw) {
  auto num = [&](const char* key) {
    const Json* v = raw.get(key);
    if (!v || v->kind != Json::Number) throw ConfigError(std::string("config.json: '") + key + "' must be a number");
    return v->number;
  };
  const double H = num("hidden_size"), V = num("vocab_size"), heads = num("heads"), kv = num("kv_heads"), d = num("head_dim");
  const double inter = num("inter"), max_pos = num("max_positions"), eps = num("eps"), theta = num("theta"), window = num("window");
  const double factor = num("rope_factor"), scale = num("scale");
  const PartSpecPtr norm = make_part("rmsnorm", {{"size", H}, {"eps", eps}});
  const PartSpecPtr head_norm = make_part("rmsnorm", {{"size", d}, {"eps", eps}});
  const PartSpecPtr rope = make_part("rotary", {{"head_dim", d}, {"rotary_dim", d}, {"theta", theta}, {"max_positions", max_pos}});
  const PartSpecPtr toy_rope = make_part("toy_scaled_half_rotary", {{"rotary_dim", d / 2}, {"theta", theta}, {"factor", factor}, {"max_positions", max_pos}});
  auto attention = [&](double win, std::map<std::string, PartSpecPtr> parts) {
    return make_part("attention", {{"hidden_size", H}, {"num_heads", heads}, {"num_kv_heads", kv}, {"head_dim", d}, {"scale", scale}, {"window", win}},
                     std::move(parts));
  };
  const PartSpecPtr ffn = make_part("swiglu", {{"hidden_size", H}, {"intermediate_size", inter}});
  const std::vector<PartSpecPtr> mixers = {attention(0, {{"q_norm", head_norm}, {"k_norm", head_norm}, {"position", rope}}),
                                           make_part("toy_carry", {{"hidden_size", H}, {"eps", eps}}),
                                           attention(window, {{"position", toy_rope}})};
  const std::vector<std::vector<std::string>> mixer_params = {
      {"q_proj.weight", "k_proj.weight", "v_proj.weight", "o_proj.weight", "q_norm.weight", "k_norm.weight"},
      {"in_proj.weight", "gain"},
      {"q_proj.weight", "k_proj.weight", "v_proj.weight", "o_proj.weight"}};
  ModelSpec spec;
  spec.architecture = "ToyNativeHybridForCausalLM";
  spec.vocab_size = (int64_t)V;
  spec.hidden_size = (int64_t)H;
  spec.max_positions = (int64_t)max_pos;
  spec.embedding = make_part("token_embedding", {{"vocab_size", V}, {"hidden_size", H}});
  spec.final_norm = norm;
  spec.head = make_part("linear_head", {{"vocab_size", V}, {"hidden_size", H}, {"tied", 0.0}});
  for (size_t i = 0; i < mixers.size(); ++i) {
    const std::string p = "l" + std::to_string(i) + ".";
    LayerSpec l;
    l.block = "prenorm";
    l.mixer = mixers[i];
    l.feed_forward = ffn;
    l.norms = {{"input", norm}, {"post_mixer", norm}};
    l.names = {{"norms.input.weight", p + "n1"}, {"norms.post_mixer.weight", p + "n2"}};
    for (const std::string& name : mixer_params[i]) l.names["mixer." + name] = p + "mixer." + name;
    for (const char* name : {"gate_proj.weight", "up_proj.weight", "down_proj.weight"}) l.names[std::string("feed_forward.") + name] = p + "ffn." + name;
    spec.layers.push_back(std::move(l));
  }
  spec.schedule = {{0, -1}, {1, -1}, {2, -1}, {0, -1}, {2, 2}};
  spec.names = {{"embedding.weight", "emb"}, {"final_norm.weight", "norm"}, {"head.weight", "head"}};
  return spec;
}

}  // namespace

extern "C" void vosti_plugin_register(void) {
  register_part("position", "toy_scaled_half_rotary",
                [](const PartSpec& s, Kernels& k) { return std::unique_ptr<Part>(new ScaledHalfRotary(s, k)); });
  register_architecture("ToyScaledRopeForCausalLM", "toy_scaled_rope", toy_scaled_rope);
  register_part("mixer", "toy_carry", [](const PartSpec& s, Kernels& k) { return std::unique_ptr<Part>(new Carry(s, k)); });
  register_architecture("ToyNativeHybridForCausalLM", "toy_native_hybrid", toy_native_hybrid);
}
