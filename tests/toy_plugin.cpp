// A plugin of the native engine, for tests: a position encoding and an architecture that the engine's own files
// know nothing of.  Compiled by the test with the host compiler against csrc/engine/parts.h and loaded with
// load_plugin(); it is a toy, never a model of anyone's.
//
// "toy_scaled_half_rotary": a half-rotation of the first half of each head only, at positions scaled down by
// `factor` (angle = inv_freq[j] * p / factor, inv_freq over the rotated width).  It offers no tables to the
// mixer, so the attention part cannot run it inside its fused launch and has to call apply().
//
// "ToyScaledRopeForCausalLM": the Qwen3 decoder with that encoding in every layer; config.json has the Qwen3
// keys and "toy_rope_factor".
#include <cmath>

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

}  // namespace

extern "C" void vosti_plugin_register(void) {
  register_part("position", "toy_scaled_half_rotary",
                [](const PartSpec& s, Kernels& k) { return std::unique_ptr<Part>(new ScaledHalfRotary(s, k)); });
  register_architecture("ToyScaledRopeForCausalLM", "toy_scaled_rope", toy_scaled_rope);
}
