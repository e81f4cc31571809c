// What a model is made of, as data, and the registry from an architecture's name to the function that
// writes that description from config.json.  Nothing below a configuration knows an architecture's name.
#pragma once
#include <cstdint>
#include <functional>
#include <map>
#include <memory>
#include <string>
#include <vector>

#include "json.h"

namespace vosti {

struct ConfigError : std::runtime_error {
  using std::runtime_error::runtime_error;
};

// A part chosen by `kind` from its category's registry, with its sizes and constants and the parts below it.
struct PartSpec {
  std::string kind;
  std::map<std::string, double> numbers;
  std::map<std::string, std::shared_ptr<const PartSpec>> parts;

  double number(const std::string& name) const;
  double number(const std::string& name, double otherwise) const;
  int64_t integer(const std::string& name) const;
  int64_t integer(const std::string& name, int64_t otherwise) const;
  const PartSpec* part(const std::string& name) const;     // nullptr if absent
};
using PartSpecPtr = std::shared_ptr<const PartSpec>;

// One layer: how its parts are arranged (`block`) and which parts they are.  `names` maps a parameter
// path inside the layer ("mixer.q_proj.weight", "norms.input.weight") to the tensor's name in the files.
struct LayerSpec {
  std::string block;
  PartSpecPtr mixer, feed_forward;
  std::map<std::string, PartSpecPtr> norms;
  std::map<std::string, std::string> names;
};

// One execution of a layer; a layer may be named by several entries.  cache_from >= 0: the index of an
// earlier entry whose cache this execution reads instead of writing one of its own.
struct ScheduleEntry {
  int layer = 0;
  int cache_from = -1;
};

struct ModelSpec {
  std::string architecture;
  int64_t vocab_size = 0, hidden_size = 0, max_positions = 0;
  PartSpecPtr embedding, final_norm, head;
  std::vector<LayerSpec> layers;
  std::vector<ScheduleEntry> schedule;
  std::map<std::string, std::string> names;          // "embedding.weight", "final_norm.weight", "head.weight"
  std::vector<std::string> ignored_names;            // tensors a checkpoint may hold although the model does not use them
  std::string config_json = "{}";                    // the typed configuration the architecture read, as a JSON object
  void validate() const;
};

// A number as JSON writes it: whole numbers without a fraction, others with the 17 digits that give the
// same 64-bit value back.
std::string json_number(double v);
std::string json_string(const std::string& s);
// The description as one JSON object: {"architecture", "vocab_size", "hidden_size", "max_positions", "config",
// "embedding", "final_norm", "head" (parts: {"kind", "numbers", "parts"}), "layers" ([{"block", "mixer",
// "feed_forward", "norms", "names"}]), "schedule" ([[layer, cache_from]]), "names", "ignored_names"}.  Hosts in
// other languages read the rules of an architecture from this instead of writing them again.
std::string model_spec_json(const ModelSpec& spec);

using ArchitectureFactory = std::function<ModelSpec(const Json& config)>;
void register_architecture(const std::string& name, const std::string& model_type, ArchitectureFactory make);
// model_type -> architecture name, for the command line's --family.
std::map<std::string, std::string> model_types();
// Reads DIR/config.json, finds the architecture by its "architectures" entry and returns its description.
ModelSpec model_spec_from_dir(const std::string& model_dir);
ModelSpec model_spec_from_config(const Json& config);
// Whether the configuration names an architecture of this registry (by "architectures", else by "model_type").
bool architecture_known(const Json& config);
// Registers the architectures that are built into this program; safe to call more than once.
void register_builtin_architectures();

}  // namespace vosti
