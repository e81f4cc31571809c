#include "spec.h"

#include <cmath>

#include "safetensors.h"

namespace vosti {

double PartSpec::number(const std::string& name) const {
  auto it = numbers.find(name);
  if (it == numbers.end()) throw ConfigError("part '" + kind + "' has no parameter '" + name + "'");
  return it->second;
}
double PartSpec::number(const std::string& name, double otherwise) const {
  auto it = numbers.find(name);
  return it == numbers.end() ? otherwise : it->second;
}
int64_t PartSpec::integer(const std::string& name) const {
  const double v = number(name);
  if (v != std::floor(v)) throw ConfigError("part '" + kind + "': parameter '" + name + "' must be an integer");
  return (int64_t)v;
}
int64_t PartSpec::integer(const std::string& name, int64_t otherwise) const {
  return numbers.count(name) ? integer(name) : otherwise;
}
const PartSpec* PartSpec::part(const std::string& name) const {
  auto it = parts.find(name);
  return it == parts.end() ? nullptr : it->second.get();
}

void ModelSpec::validate() const {
  for (size_t i = 0; i < schedule.size(); ++i) {
    const ScheduleEntry& e = schedule[i];
    if (e.layer < 0 || e.layer >= (int)layers.size())
      throw ConfigError("schedule entry " + std::to_string(i) + " names layer " + std::to_string(e.layer) + ", but there are " +
                        std::to_string(layers.size()) + " layers");
    if (e.cache_from >= 0) {
      if (e.cache_from >= (int)i)
        throw ConfigError("schedule entry " + std::to_string(i) + " reads the cache of entry " + std::to_string(e.cache_from) +
                          ", which does not run before it");
      if (schedule[e.cache_from].cache_from >= 0)
        throw ConfigError("schedule entry " + std::to_string(i) + " reads the cache of entry " + std::to_string(e.cache_from) +
                          ", which has none of its own");
    }
  }
}

namespace {
struct Registered {
  std::string model_type;
  ArchitectureFactory make;
};
std::map<std::string, Registered>& registry() {
  static std::map<std::string, Registered> r;
  return r;
}
}  // namespace

void register_architecture(const std::string& name, const std::string& model_type, ArchitectureFactory make) {
  if (registry().count(name)) throw ConfigError("architecture '" + name + "' is registered twice");
  registry()[name] = {model_type, std::move(make)};
}

std::map<std::string, std::string> model_types() {
  std::map<std::string, std::string> out;
  for (const auto& r : registry()) out[r.second.model_type] = r.first;
  return out;
}

ModelSpec model_spec_from_config(const Json& config) {
  if (config.kind != Json::Object) throw ConfigError("config.json must hold an object");
  // The first entry of "architectures", else a registered "model_type".
  std::string name;
  const Json* archs = config.get("architectures");
  const Json* mt = config.get("model_type");
  if (archs && archs->kind == Json::Array && !archs->items.empty() && archs->items[0].kind == Json::String) {
    name = archs->items[0].text;
  } else if (mt && mt->kind == Json::String && model_types().count(mt->text)) {
    name = model_types()[mt->text];
  } else {
    throw ConfigError("config.json names no architecture (key 'architectures') and no known 'model_type'");
  }
  auto it = registry().find(name);
  if (it == registry().end()) {
    std::string known;
    for (const auto& r : registry()) known += (known.empty() ? "" : ", ") + r.first;
    throw ConfigError("unknown architecture '" + name + "'; registered: " + (known.empty() ? "none" : known));
  }
  ModelSpec spec = it->second.make(config);
  spec.validate();
  return spec;
}

ModelSpec model_spec_from_dir(const std::string& model_dir) {
  const std::string path = model_dir + "/config.json";
  if (!file_exists(path)) throw ConfigError(path + " is missing");
  try {
    return model_spec_from_config(Json::parse(read_text_file(path)));
  } catch (const JsonError& e) {
    throw ConfigError(path + ": " + e.what());
  }
}

}  // namespace vosti
