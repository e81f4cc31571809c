// The typed configuration of the Qwen3 dense decoder and its description as parts.  An architecture that is a
// variation of this one (another part kind in some place) can start from these two functions.
#pragma once
#include "spec.h"

namespace vosti {

struct Qwen3Config {
  int64_t vocab_size = 0, hidden_size = 0, intermediate_size = 0, num_hidden_layers = 0, num_attention_heads = 0, num_key_value_heads = 0,
          head_dim = 0, max_position_embeddings = 0;
  double rms_norm_eps = 0, rope_theta = 0;
  bool tie_word_embeddings = false;
  std::string to_json() const;
};

// Reads and checks the keys of config.json; every error names the key.
Qwen3Config qwen3_config(const Json& raw);
ModelSpec qwen3_model_spec(const Qwen3Config& config);

}  // namespace vosti
