// The Qwen3 dense decoder, from its config.json keys to a description of parts.
//
// The key set and the rules are those of the reference's profile projection
// (python/vosti_kernels/model_families/qwen3/profile.py:41-61 for the keys, :129-164 for the rules; typed
// twin src/boundary/model_families/qwen3/config.rs:9-18).  The reference additionally demands equality
// with one of two sealed profiles and fixes eps and theta (qwen3/physical.py:29-32); here every valid
// geometry is admitted and both are parameters.
#include <cmath>

#include "qwen3.h"

namespace vosti {
namespace {

const Json* present(const Json& raw, const std::string& key) { return raw.get(key); }

int64_t pos_int(const Json& raw, const std::string& key, int64_t otherwise = -1) {
  const Json* v = present(raw, key);
  if (!v) {
    if (otherwise >= 0) return otherwise;
    throw ConfigError("config.json: required key '" + key + "' is missing");
  }
  if (!v->is_int() || v->as_int() <= 0) throw ConfigError("config.json: '" + key + "' must be a positive integer");
  return v->as_int();
}

double pos_float(const Json* v, const std::string& key) {
  if (!v) throw ConfigError("config.json: required key '" + key + "' is missing");
  if (v->kind != Json::Number || !std::isfinite(v->number) || v->number <= 0)
    throw ConfigError("config.json: '" + key + "' must be a finite positive number");
  return v->number;
}

bool is_false_or_absent(const Json& raw, const std::string& key) {
  const Json* v = present(raw, key);
  return !v || (v->kind == Json::Bool && !v->boolean);
}

std::string rope_type_of(const Json& j) {
  if (const Json* t = j.get("rope_type")) return t->text;
  if (const Json* t = j.get("type")) return t->text;
  return "";
}

PartSpecPtr part(std::string kind, std::map<std::string, double> numbers, std::map<std::string, PartSpecPtr> parts = {}) {
  auto p = std::make_shared<PartSpec>();
  p->kind = std::move(kind);
  p->numbers = std::move(numbers);
  p->parts = std::move(parts);
  return p;
}

}  // namespace

Qwen3Config qwen3_config(const Json& raw) {
  if (const Json* mt = present(raw, "model_type"))
    if (mt->text != "qwen3") throw ConfigError("config.json: 'model_type' is '" + mt->text + "', expected 'qwen3'");
  const int64_t hidden = pos_int(raw, "hidden_size");
  const int64_t heads = pos_int(raw, "num_attention_heads");
  const int64_t kv_heads = pos_int(raw, "num_key_value_heads", heads);
  int64_t head_dim;
  if (present(raw, "head_dim")) {
    head_dim = pos_int(raw, "head_dim");
  } else {
    if (hidden % heads) throw ConfigError("config.json: 'head_dim' is absent and 'hidden_size' is not a multiple of 'num_attention_heads'");
    head_dim = hidden / heads;
  }
  if (heads % kv_heads)
    throw ConfigError("config.json: 'num_attention_heads' (" + std::to_string(heads) + ") must be a multiple of 'num_key_value_heads' (" +
                      std::to_string(kv_heads) + ")");
  if (head_dim % 2) throw ConfigError("config.json: 'head_dim' (" + std::to_string(head_dim) + ") must be even");
  if (const Json* act = present(raw, "hidden_act"))
    if (act->text != "silu") throw ConfigError("config.json: 'hidden_act' is '" + act->text + "'; this architecture uses 'silu'");
  if (!is_false_or_absent(raw, "attention_bias")) throw ConfigError("config.json: 'attention_bias' must be false");
  if (const Json* drop = present(raw, "attention_dropout"))
    if (drop->kind != Json::Number || drop->number != 0.0) throw ConfigError("config.json: 'attention_dropout' must be 0");
  if (!is_false_or_absent(raw, "use_sliding_window"))
    throw ConfigError("config.json: 'use_sliding_window' must be false: this architecture attends to all keys");
  const Json* layer_types = present(raw, "layer_types");
  if (layer_types)
    for (const Json& t : layer_types->items)
      if (t.text != "full_attention") throw ConfigError("config.json: 'layer_types' must name 'full_attention' for every layer");
  const Json* theta = present(raw, "rope_theta");
  const Json* scaling = present(raw, "rope_scaling");
  if (const Json* rp = present(raw, "rope_parameters")) {
    if (rp->kind == Json::Object) {
      if (!theta) theta = rp->get("rope_theta");
      const Json* rt = rp->get("rope_type");
      if (rt && rt->text != "default") scaling = rp;
    }
  }
  if (scaling && !(scaling->kind == Json::Object && rope_type_of(*scaling) == "default"))
    throw ConfigError("config.json: 'rope_scaling' must be null: only the default rotary encoding is built");
  bool tie = false;
  if (const Json* t = present(raw, "tie_word_embeddings")) {
    if (t->kind != Json::Bool) throw ConfigError("config.json: 'tie_word_embeddings' must be true or false");
    tie = t->boolean;
  }
  // A model without layers is lm_head(rms_norm(embed)) (src/exec/dense_swiglu_model.rs:276-359).
  const Json* nl = present(raw, "num_hidden_layers");
  if (!nl) throw ConfigError("config.json: required key 'num_hidden_layers' is missing");
  if (!nl->is_int() || nl->as_int() < 0) throw ConfigError("config.json: 'num_hidden_layers' must be an integer, zero or more");
  const int64_t layers = nl->as_int();
  if (layer_types && (int64_t)layer_types->items.size() != layers)
    throw ConfigError("config.json: 'layer_types' must have one entry per layer");
  Qwen3Config c;
  c.vocab_size = pos_int(raw, "vocab_size");
  c.hidden_size = hidden;
  c.intermediate_size = pos_int(raw, "intermediate_size");
  c.num_hidden_layers = layers;
  c.num_attention_heads = heads;
  c.num_key_value_heads = kv_heads;
  c.head_dim = head_dim;
  c.max_position_embeddings = pos_int(raw, "max_position_embeddings");
  c.rms_norm_eps = pos_float(present(raw, "rms_norm_eps"), "rms_norm_eps");
  c.rope_theta = pos_float(theta, "rope_theta");
  c.tie_word_embeddings = tie;
  return c;
}

std::string Qwen3Config::to_json() const {
  return "{\"vocab_size\": " + std::to_string(vocab_size) + ", \"hidden_size\": " + std::to_string(hidden_size) +
         ", \"intermediate_size\": " + std::to_string(intermediate_size) + ", \"num_hidden_layers\": " + std::to_string(num_hidden_layers) +
         ", \"num_attention_heads\": " + std::to_string(num_attention_heads) + ", \"num_key_value_heads\": " + std::to_string(num_key_value_heads) +
         ", \"head_dim\": " + std::to_string(head_dim) + ", \"max_position_embeddings\": " + std::to_string(max_position_embeddings) +
         ", \"rms_norm_eps\": " + json_number(rms_norm_eps) + ", \"rope_theta\": " + json_number(rope_theta) +
         ", \"tie_word_embeddings\": " + (tie_word_embeddings ? "true" : "false") + "}";
}

// Pre-norm blocks of attention and SwiGLU (src/exec/dense_swiglu_decoder.rs:43-441), every layer alike,
// run once each in order (src/exec/dense_swiglu_model.rs:131-1041).
ModelSpec qwen3_model_spec(const Qwen3Config& c) {
  const int64_t hidden = c.hidden_size, heads = c.num_attention_heads, kv_heads = c.num_key_value_heads, head_dim = c.head_dim;
  const int64_t vocab = c.vocab_size, inter = c.intermediate_size, max_pos = c.max_position_embeddings, layers = c.num_hidden_layers;
  const double eps = c.rms_norm_eps, rope_theta = c.rope_theta;
  const bool tie = c.tie_word_embeddings;
  const PartSpecPtr norm = part("rmsnorm", {{"size", (double)hidden}, {"eps", eps}});
  const PartSpecPtr head_norm = part("rmsnorm", {{"size", (double)head_dim}, {"eps", eps}});
  const PartSpecPtr rope = part("rotary", {{"head_dim", (double)head_dim}, {"rotary_dim", (double)head_dim}, {"theta", rope_theta},
                                           {"max_positions", (double)max_pos}});
  const PartSpecPtr mixer = part("attention",
                                 {{"hidden_size", (double)hidden}, {"num_heads", (double)heads}, {"num_kv_heads", (double)kv_heads},
                                  {"head_dim", (double)head_dim}, {"scale", std::pow((double)head_dim, -0.5)}, {"window", 0.0}},
                                 {{"q_norm", head_norm}, {"k_norm", head_norm}, {"position", rope}});
  const PartSpecPtr ffn = part("swiglu", {{"hidden_size", (double)hidden}, {"intermediate_size", (double)inter}});

  ModelSpec spec;
  spec.architecture = "Qwen3ForCausalLM";
  spec.vocab_size = vocab;
  spec.hidden_size = hidden;
  spec.max_positions = max_pos;
  spec.embedding = part("token_embedding", {{"vocab_size", (double)vocab}, {"hidden_size", (double)hidden}});
  spec.final_norm = norm;
  spec.head = part("linear_head", {{"vocab_size", (double)vocab}, {"hidden_size", (double)hidden}, {"tied", tie ? 1.0 : 0.0}});
  for (int64_t i = 0; i < layers; ++i) {
    const std::string p = "model.layers." + std::to_string(i) + ".";
    LayerSpec l;
    l.block = "prenorm";
    l.mixer = mixer;
    l.feed_forward = ffn;
    l.norms = {{"input", norm}, {"post_mixer", norm}};
    l.names = {{"norms.input.weight", p + "input_layernorm.weight"},
               {"norms.post_mixer.weight", p + "post_attention_layernorm.weight"},
               {"mixer.q_proj.weight", p + "self_attn.q_proj.weight"},
               {"mixer.k_proj.weight", p + "self_attn.k_proj.weight"},
               {"mixer.v_proj.weight", p + "self_attn.v_proj.weight"},
               {"mixer.o_proj.weight", p + "self_attn.o_proj.weight"},
               {"mixer.q_norm.weight", p + "self_attn.q_norm.weight"},
               {"mixer.k_norm.weight", p + "self_attn.k_norm.weight"},
               {"feed_forward.gate_proj.weight", p + "mlp.gate_proj.weight"},
               {"feed_forward.up_proj.weight", p + "mlp.up_proj.weight"},
               {"feed_forward.down_proj.weight", p + "mlp.down_proj.weight"}};
    spec.layers.push_back(std::move(l));
    spec.schedule.push_back({(int)i, -1});
  }
  // A tied head is the embedding table itself (python/vosti_kernels/model_families/qwen3/physical.py:131-134);
  // a checkpoint that stores an lm_head.weight beside it is tolerated.
  spec.names = {{"embedding.weight", "model.embed_tokens.weight"},
                {"final_norm.weight", "model.norm.weight"},
                {"head.weight", tie ? "model.embed_tokens.weight" : "lm_head.weight"}};
  if (tie) spec.ignored_names = {"lm_head.weight"};
  spec.config_json = c.to_json();
  return spec;
}

void register_builtin_architectures() {
  static bool done = false;
  if (done) return;
  done = true;
  register_architecture("Qwen3ForCausalLM", "qwen3", [](const Json& raw) { return qwen3_model_spec(qwen3_config(raw)); });
}

}  // namespace vosti
