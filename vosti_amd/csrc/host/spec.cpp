#include "spec.h"

#include <cmath>
#include <cstdio>

#include "files.h"

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

std::string json_number(double v) {
  char buf[40];
  if (v == std::floor(v) && std::fabs(v) < 9.0e15) std::snprintf(buf, sizeof buf, "%lld", (long long)v);
  else std::snprintf(buf, sizeof buf, "%.17g", v);
  return buf;
}

std::string json_string(const std::string& s) {
  std::string out = "\"";
  for (char c : s) {
    if (c == '"' || c == '\\') out += '\\';
    if ((unsigned char)c < 0x20) {
      char buf[8];
      std::snprintf(buf, sizeof buf, "\\u%04x", c);
      out += buf;
    } else {
      out += c;
    }
  }
  return out + "\"";
}

namespace {
std::string names_json(const std::map<std::string, std::string>& names) {
  std::string out = "{";
  for (const auto& n : names) out += (out.size() > 1 ? ", " : "") + json_string(n.first) + ": " + json_string(n.second);
  return out + "}";
}

std::string part_json(const PartSpec& p) {
  std::string out = "{\"kind\": " + json_string(p.kind) + ", \"numbers\": {";
  bool first = true;
  for (const auto& n : p.numbers) {
    out += (first ? "" : ", ") + json_string(n.first) + ": " + json_number(n.second);
    first = false;
  }
  out += "}, \"parts\": {";
  first = true;
  for (const auto& c : p.parts) {
    out += (first ? "" : ", ") + json_string(c.first) + ": " + part_json(*c.second);
    first = false;
  }
  return out + "}}";
}
}  // namespace

std::string model_spec_json(const ModelSpec& spec) {
  std::string out = "{\"architecture\": " + json_string(spec.architecture) + ", \"vocab_size\": " + std::to_string(spec.vocab_size) +
                    ", \"hidden_size\": " + std::to_string(spec.hidden_size) + ", \"max_positions\": " + std::to_string(spec.max_positions) +
                    ", \"config\": " + spec.config_json + ", \"embedding\": " + part_json(*spec.embedding) +
                    ", \"final_norm\": " + part_json(*spec.final_norm) + ", \"head\": " + part_json(*spec.head) + ", \"layers\": [";
  // Layers that are alike are written once: "same_as" names the first layer with the same parts, so that a deep
  // model's description stays short; the tensor names are each layer's own.
  for (size_t i = 0; i < spec.layers.size(); ++i) {
    const LayerSpec& l = spec.layers[i];
    out += i ? ", {" : "{";
    size_t same = i;
    for (size_t j = 0; j < i; ++j)
      if (spec.layers[j].block == l.block && spec.layers[j].mixer == l.mixer && spec.layers[j].feed_forward == l.feed_forward &&
          spec.layers[j].norms == l.norms) {
        same = j;
        break;
      }
    if (same != i) {
      out += "\"same_as\": " + std::to_string(same);
    } else {
      out += "\"block\": " + json_string(l.block) + ", \"mixer\": " + part_json(*l.mixer) + ", \"feed_forward\": " + part_json(*l.feed_forward) +
             ", \"norms\": {";
      bool first = true;
      for (const auto& n : l.norms) {
        out += (first ? "" : ", ") + json_string(n.first) + ": " + part_json(*n.second);
        first = false;
      }
      out += "}";
    }
    out += ", \"names\": " + names_json(l.names) + "}";
  }
  out += "], \"schedule\": [";
  for (size_t i = 0; i < spec.schedule.size(); ++i)
    out += (i ? ", [" : "[") + std::to_string(spec.schedule[i].layer) + ", " + std::to_string(spec.schedule[i].cache_from) + "]";
  out += "], \"names\": " + names_json(spec.names) + ", \"ignored_names\": [";
  for (size_t i = 0; i < spec.ignored_names.size(); ++i) out += (i ? ", " : "") + json_string(spec.ignored_names[i]);
  return out + "]}";
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

// The first entry of "architectures", else a registered "model_type"; empty if neither is there.
static std::string architecture_name(const Json& config) {
  const Json* archs = config.get("architectures");
  const Json* mt = config.get("model_type");
  if (archs && archs->kind == Json::Array && !archs->items.empty() && archs->items[0].kind == Json::String) return archs->items[0].text;
  if (mt && mt->kind == Json::String && model_types().count(mt->text)) return model_types()[mt->text];
  return "";
}

bool architecture_known(const Json& config) { return config.kind == Json::Object && registry().count(architecture_name(config)) > 0; }

ModelSpec model_spec_from_config(const Json& config) {
  if (config.kind != Json::Object) throw ConfigError("config.json must hold an object");
  const std::string name = architecture_name(config);
  if (name.empty()) throw ConfigError("config.json names no architecture (key 'architectures') and no known 'model_type'");
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
