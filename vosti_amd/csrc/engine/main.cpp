// Command line of the native engine, in the manner of the reference's engine example.
//
//     vosti_engine [--kind engine] --family qwen3 [--] [options]
//     vosti_engine --kind describe --model-path DIR      (what config.json and the weight files say; no GPU)
//
// The reference starts its engine example through scripts/launch.py --kind engine --family qwen3
// (scripts/launch.py:17-55) and configures it by environment variables
// (examples/support/engine_setup.rs:57-69, 110-118; examples/support/engine_serving.rs:75-231).  The same
// variables mean the same here; each also has an option, which wins:
//
//     MODEL_PATH                 --model-path          model folder (required)
//     CUDA_DEVICE                --device              only cuda:0 exists here
//     VOSTI_PROMPT_IDS           --prompt-ids          comma-separated token ids (default "9707")
//     VOSTI_MAX_TOKENS           --max-tokens          new tokens (default 8)
//     VOSTI_IGNORE_EOS           --ignore-eos          presence: do not stop on end tokens
//     VOSTI_NUM_BLOCKS           --num-blocks          cache pages (default 32)
//     VOSTI_MAX_SEQS             --max-seqs            rows per step (default: the batch size)
//     VOSTI_MAX_BATCHED_TOKENS   --max-batched-tokens  tokens per step (default 4096)
//     VOSTI_CUDA_GRAPH           --graphs              0/1: replay decode steps from recorded HIP graphs
//     VOSTI_OUTPUT_TOKENS        --output-tokens       write "index<TAB>ids" lines to this file
//     VOSTI_BENCH_INPUT          --bench-input         TSV of MAX_TOKENS<TAB>IDS[<TAB>ARRIVAL_STEP] requests
//     VOSTI_BENCH_WARMUP_INPUT   --bench-warmup-input  a TSV of other requests, served first by the same engine
//     VOSTI_BENCH_GRAPH_PRIMER_INPUT --bench-graph-primer-input  a third TSV, served before the warm-up so that the
//                                                      recordings of its decode steps exist before anything is timed
//     VOSTI_BENCH_CALLS          --bench-calls         JSON of several calls served one after the other by one engine
//     VOSTI_BENCH_CALL_RESULTS   --bench-call-results  where their records go (a new JSON file)
//     VOSTI_LOGITS_DIGEST                              a file that gets "row sha256" for every sampled logits row
//     VOSTI_LOGITS_OBSERVER_DIR                        a folder that gets every sampled logits row as float32 .npy and an index
//     VOSTI_MAX_MODEL_LEN        --max-model-len       longest prompt plus output (default: the model's positions)
//     VOSTI_ENGINE_STEP_TRACE    --step-trace          append one JSON line per step to this file
//
// Options without a counterpart in the reference: VOSTI_DTYPE / --dtype (bfloat16, float32),
// VOSTI_TEMPERATURE / --temperature, VOSTI_SEED / --seed, VOSTI_PAGE_SIZE / --page-size,
// VOSTI_PREFIX_CACHE / --prefix-cache (0, 1), VOSTI_LIB_DIR / --lib-dir (where the kernel libraries lie;
// default: beside this program), VOSTI_RANDOM_WEIGHTS / --random-weights SEED (the folder needs config.json
// only; the weights are those of the Python launcher's random-model kind for that seed), VOSTI_STEP_TIMES /
// --step-times FILE (one line "rows tokens sampled ms" per engine step), VOSTI_PLUGINS (paths, colon-separated) /
// --plugin PATH (may be given more than once): shared libraries that register part kinds and architectures of
// their own before the model folder is read.  End tokens come from generation_config.json's eos_token_id (one to three
// ids: python/vosti_kernels/serving_workload.py:78-108); without that file there are none.  It prints
// MODEL_OUTPUT_TOKEN_IDS=[...] like the reference, or a BENCH batch=... tok_s=... line for prepared requests.
#include <unistd.h>

#include <algorithm>
#include <chrono>
#include <climits>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <iostream>
#include <sstream>

#include "engine.h"

using namespace vosti;

namespace {

struct Usage : std::runtime_error {
  using std::runtime_error::runtime_error;
};

struct Prepared {
  int max_tokens;
  std::vector<int32_t> ids;
  int arrival;
};

std::string env_or(const char* name, const std::string& otherwise) {
  const char* v = std::getenv(name);
  return (v && *v) ? v : otherwise;
}

long to_int(const std::string& text, const std::string& what) {
  char* end = nullptr;
  const long v = std::strtol(text.c_str(), &end, 10);
  if (text.empty() || *end) throw Usage(what + " must be an integer, got '" + text + "'");
  return v;
}

std::vector<int32_t> parse_ids(const std::string& text) {
  std::vector<int32_t> ids;
  std::string item;
  std::string clean;
  for (char c : text)
    if (c != ' ') clean += c;
  std::stringstream ss(clean);
  while (std::getline(ss, item, ','))
    if (!item.empty()) ids.push_back((int32_t)to_int(item, "prompt ids"));
  if (ids.empty()) throw Usage("the prompt is empty");
  return ids;
}

// MAX_TOKENS<TAB>IDS[<TAB>ARRIVAL_STEP] per line; '#' starts a comment (examples/support/engine_benchmark.rs:79-165).
std::vector<Prepared> parse_prepared(const std::string& path) {
  std::ifstream f(path);
  if (!f) throw Usage("cannot read " + path);
  std::vector<Prepared> out;
  std::string line;
  for (int n = 1; std::getline(f, line); ++n) {
    const size_t first = line.find_first_not_of(" \t\r");
    if (first == std::string::npos || line[first] == '#') continue;
    std::vector<std::string> fields;
    std::stringstream ss(line);
    std::string field;
    while (std::getline(ss, field, '\t')) fields.push_back(field);
    if (fields.size() != 2 && fields.size() != 3) throw Usage(path + ":" + std::to_string(n) + ": expected MAX_TOKENS<TAB>IDS[<TAB>ARRIVAL_STEP]");
    out.push_back({(int)to_int(fields[0], "MAX_TOKENS"), parse_ids(fields[1]), fields.size() == 3 ? (int)to_int(fields[2], "ARRIVAL_STEP") : 0});
  }
  if (out.empty()) throw Usage(path + " holds no requests");
  return out;
}

std::vector<int32_t> eos_ids(const std::string& model_dir) {
  const std::string path = model_dir + "/generation_config.json";
  std::vector<int32_t> ids;
  if (!file_exists(path)) return ids;
  const Json j = Json::parse(read_text_file(path));
  const Json* v = j.get("eos_token_id");
  if (!v) return ids;
  if (v->kind == Json::Number) ids.push_back((int32_t)v->as_int());
  else
    for (const Json& i : v->items) ids.push_back((int32_t)i.as_int());
  if (ids.empty() || ids.size() > 3) throw Usage("generation_config.json: 'eos_token_id' must hold one to three ids");
  return ids;
}

std::string self_dir() {
  char buf[PATH_MAX];
  const ssize_t n = readlink("/proc/self/exe", buf, sizeof(buf) - 1);
  if (n <= 0) return ".";
  buf[n] = 0;
  std::string p(buf);
  return p.substr(0, p.find_last_of('/'));
}

std::string id_list(const std::vector<int32_t>& ids, const char* sep) {
  std::string s;
  for (size_t i = 0; i < ids.size(); ++i) s += (i ? sep : "") + std::to_string(ids[i]);
  return s;
}

std::vector<std::string> split_list(const std::string& text, char sep) {
  std::vector<std::string> out;
  std::stringstream ss(text);
  std::string item;
  while (std::getline(ss, item, sep))
    if (!item.empty()) out.push_back(item);
  return out;
}

struct Options {
  std::string kind = "engine", family;
  std::string model_path = env_or("MODEL_PATH", ""), device = env_or("CUDA_DEVICE", "cuda:0");
  std::string prompt_ids = env_or("VOSTI_PROMPT_IDS", "9707");
  long max_tokens = to_int(env_or("VOSTI_MAX_TOKENS", "8"), "VOSTI_MAX_TOKENS");
  bool ignore_eos = std::getenv("VOSTI_IGNORE_EOS") != nullptr;
  long num_blocks = to_int(env_or("VOSTI_NUM_BLOCKS", "32"), "VOSTI_NUM_BLOCKS");
  long max_seqs = to_int(env_or("VOSTI_MAX_SEQS", "0"), "VOSTI_MAX_SEQS");
  long max_batched_tokens = to_int(env_or("VOSTI_MAX_BATCHED_TOKENS", "4096"), "VOSTI_MAX_BATCHED_TOKENS");
  long graphs = to_int(env_or("VOSTI_CUDA_GRAPH", "0"), "VOSTI_CUDA_GRAPH");
  std::string output_tokens = env_or("VOSTI_OUTPUT_TOKENS", ""), bench_input = env_or("VOSTI_BENCH_INPUT", "");
  std::string bench_warmup_input = env_or("VOSTI_BENCH_WARMUP_INPUT", "");
  std::string bench_graph_primer_input = env_or("VOSTI_BENCH_GRAPH_PRIMER_INPUT", "");
  std::string bench_calls = env_or("VOSTI_BENCH_CALLS", ""), bench_call_results = env_or("VOSTI_BENCH_CALL_RESULTS", "");
  long max_model_len = to_int(env_or("VOSTI_MAX_MODEL_LEN", "0"), "VOSTI_MAX_MODEL_LEN");
  std::string step_trace = env_or("VOSTI_ENGINE_STEP_TRACE", ""), dtype = env_or("VOSTI_DTYPE", "bfloat16");
  double temperature = std::atof(env_or("VOSTI_TEMPERATURE", "0").c_str());
  long seed = to_int(env_or("VOSTI_SEED", "0"), "VOSTI_SEED");
  long page_size = to_int(env_or("VOSTI_PAGE_SIZE", "64"), "VOSTI_PAGE_SIZE");
  long prefix_cache = to_int(env_or("VOSTI_PREFIX_CACHE", "1"), "VOSTI_PREFIX_CACHE");
  std::string lib_dir = env_or("VOSTI_LIB_DIR", "");
  std::string random_weights = env_or("VOSTI_RANDOM_WEIGHTS", ""), step_times = env_or("VOSTI_STEP_TIMES", "");
  std::vector<std::string> plugins = split_list(env_or("VOSTI_PLUGINS", ""), ':');
};

Options parse(int argc, char** argv) {
  Options o;
  for (int i = 1; i < argc; ++i) {
    std::string a = argv[i], value;
    if (a == "--") continue;
    bool has_value = false;
    const size_t eq = a.find('=');
    if (a.rfind("--", 0) == 0 && eq != std::string::npos) {
      value = a.substr(eq + 1);
      a = a.substr(0, eq);
      has_value = true;
    }
    auto val = [&]() -> std::string {
      if (has_value) return value;
      if (i + 1 >= argc) throw Usage(a + " needs a value");
      return argv[++i];
    };
    if (a == "--kind") o.kind = val();
    else if (a == "--family") o.family = val();
    else if (a == "--model-path") o.model_path = val();
    else if (a == "--device") o.device = val();
    else if (a == "--prompt-ids") o.prompt_ids = val();
    else if (a == "--max-tokens") o.max_tokens = to_int(val(), a);
    else if (a == "--ignore-eos") o.ignore_eos = true;
    else if (a == "--num-blocks") o.num_blocks = to_int(val(), a);
    else if (a == "--max-seqs") o.max_seqs = to_int(val(), a);
    else if (a == "--max-batched-tokens") o.max_batched_tokens = to_int(val(), a);
    else if (a == "--graphs") o.graphs = to_int(val(), a);
    else if (a == "--output-tokens") o.output_tokens = val();
    else if (a == "--bench-input") o.bench_input = val();
    else if (a == "--bench-warmup-input") o.bench_warmup_input = val();
    else if (a == "--bench-graph-primer-input") o.bench_graph_primer_input = val();
    else if (a == "--bench-calls") o.bench_calls = val();
    else if (a == "--bench-call-results") o.bench_call_results = val();
    else if (a == "--max-model-len") o.max_model_len = to_int(val(), a);
    else if (a == "--step-trace") o.step_trace = val();
    else if (a == "--dtype") o.dtype = val();
    else if (a == "--temperature") o.temperature = std::atof(val().c_str());
    else if (a == "--seed") o.seed = to_int(val(), a);
    else if (a == "--page-size") o.page_size = to_int(val(), a);
    else if (a == "--prefix-cache") o.prefix_cache = to_int(val(), a);
    else if (a == "--lib-dir") o.lib_dir = val();
    else if (a == "--random-weights") o.random_weights = val();
    else if (a == "--step-times") o.step_times = val();
    else if (a == "--plugin") o.plugins.push_back(val());
    else throw Usage("unknown option " + a);
  }
  return o;
}

std::string quoted(const std::string& s) {
  std::string out = "\"";
  for (char c : s) {
    if (c == '"' || c == '\\') out += '\\';
    out += c;
  }
  return out + "\"";
}

std::string shape_list(const std::vector<int64_t>& shape) {
  std::string s = "[";
  for (size_t i = 0; i < shape.size(); ++i) s += (i ? ", " : "") + std::to_string(shape[i]);
  return s + "]";
}

// --kind describe: what config.json says and what the weight files hold, as one JSON object.  It needs no GPU.
int describe(const Options& o) {
  register_builtin_architectures();
  const ModelSpec spec = model_spec_from_dir(o.model_path);
  std::string out = "{\"architecture\": " + quoted(spec.architecture) + ", \"vocab_size\": " + std::to_string(spec.vocab_size) +
                    ", \"hidden_size\": " + std::to_string(spec.hidden_size) + ", \"max_positions\": " + std::to_string(spec.max_positions) +
                    ", \"layers\": " + std::to_string(spec.layers.size()) + ", \"schedule\": " + std::to_string(spec.schedule.size());
  out += ", \"tensor_names\": [";
  std::vector<std::string> names;
  for (const auto& n : spec.names) names.push_back(n.second);
  for (const LayerSpec& l : spec.layers)
    for (const auto& n : l.names) names.push_back(n.second);
  std::sort(names.begin(), names.end());
  names.erase(std::unique(names.begin(), names.end()), names.end());
  for (size_t i = 0; i < names.size(); ++i) out += (i ? ", " : "") + quoted(names[i]);
  if (!o.random_weights.empty()) {
    // The seed of every tensor's random stream, as decimal text (they do not fit a double).
    const uint64_t seed = (uint64_t)to_int(o.random_weights, "--random-weights");
    out += "], \"tensor_seeds\": [";
    for (size_t i = 0; i < names.size(); ++i) out += (i ? ", " : "") + quoted(std::to_string(tensor_seed(seed, names[i])));
  }
  out += "], \"ignored_names\": [";
  for (size_t i = 0; i < spec.ignored_names.size(); ++i) out += (i ? ", " : "") + quoted(spec.ignored_names[i]);
  out += "]";
  if (file_exists(o.model_path + "/model.safetensors") || file_exists(o.model_path + "/model.safetensors.index.json")) {
    const Checkpoint ckpt(o.model_path);
    out += ", \"stored\": {";
    bool first = true;
    for (const auto& e : ckpt.entries()) {
      out += (first ? "" : ", ") + quoted(e.first) + ": {\"dtype\": " + quoted(e.second.dtype) + ", \"shape\": " + shape_list(e.second.shape) + "}";
      first = false;
    }
    out += "}";
  }
  std::cout << out << "}\n";
  return 0;
}

std::string ids_json(const std::vector<std::vector<int32_t>>& lists) {
  std::string s = "[";
  for (size_t i = 0; i < lists.size(); ++i) s += (i ? ", [" : "[") + id_list(lists[i], ", ") + "]";
  return s + "]";
}

// Several calls through one engine, one after the other (examples/support/engine_calls.rs:58-123):
// {"prefix_caching": bool, "calls": [{"label", "prompts" | "output_prefix_from", "max_tokens"}]}.  A call's prompts
// are given outright, or built from an earlier call's prompt, the first `count` tokens that call generated for it,
// and a suffix (:32-56).  Without prefix caching the cached pages are dropped before every call.  One record per
// call goes to the results file, and CALLS_FINISHED <n> is printed.
int run_calls(Engine& engine, const Options& o, const std::vector<int32_t>& eos) {
  const Json spec = Json::parse(read_text_file(o.bench_calls));
  const Json* calls = spec.get("calls");
  if (!calls || calls->kind != Json::Array || calls->items.empty()) throw Usage("bench calls: the file holds no calls");
  if (o.bench_call_results.empty()) throw Usage("bench calls: VOSTI_BENCH_CALL_RESULTS (or --bench-call-results) is required");
  if (file_exists(o.bench_call_results)) throw Usage("bench calls: " + o.bench_call_results + " exists already");
  const Json* pc = spec.get("prefix_caching");
  const bool prefix_caching = pc && pc->kind == Json::Bool && pc->boolean;
  std::vector<std::pair<std::vector<std::vector<int32_t>>, std::vector<std::vector<int32_t>>>> prior;
  std::string records = "[";
  RequestId base = 0;
  for (size_t index = 0; index < calls->items.size(); ++index) {
    const Json& call = calls->items[index];
    if (engine.has_unfinished()) throw Usage("bench calls: the call before did not finish");
    const int dropped = prefix_caching ? 0 : engine.cache().drop_cached();
    std::vector<std::vector<int32_t>> prompts;
    if (const Json* src = call.get("output_prefix_from")) {
      const Json *c = src->get("call"), *r = src->get("request"), *n = src->get("count");
      if (!c || !r || !n) throw Usage("bench calls: 'output_prefix_from' needs 'call', 'request' and 'count'");
      if (c->as_int() < 0 || c->as_int() >= (int64_t)prior.size()) throw Usage("bench calls: 'output_prefix_from' names a call that has not run yet");
      const auto& from = prior[(size_t)c->as_int()];
      if (r->as_int() < 0 || r->as_int() >= (int64_t)from.first.size()) throw Usage("bench calls: 'output_prefix_from' names a request that the call does not have");
      const auto& out = from.second[(size_t)r->as_int()];
      if (n->as_int() < 0 || n->as_int() > (int64_t)out.size()) throw Usage("bench calls: 'output_prefix_from' wants more tokens than were generated");
      std::vector<int32_t> query = from.first[(size_t)r->as_int()];
      query.insert(query.end(), out.begin(), out.begin() + n->as_int());
      if (const Json* suffix = src->get("suffix"))
        for (const Json& t : suffix->items) query.push_back((int32_t)t.as_int());
      prompts.push_back(std::move(query));
    } else if (const Json* ps = call.get("prompts")) {
      for (const Json& p : ps->items) {
        prompts.emplace_back();
        for (const Json& t : p.items) prompts.back().push_back((int32_t)t.as_int());
      }
    }
    const Json* mt = call.get("max_tokens");
    const int max_tokens = mt ? (int)mt->as_int() : 0;
    bool empty = prompts.empty() || max_tokens <= 0;
    for (const auto& p : prompts) empty = empty || p.empty();
    if (empty) throw Usage("bench calls: a call has an empty prompt, an empty batch or no output budget");
    setenv("VOSTI_LOGITS_OBSERVER_PHASE", ("call-" + std::to_string(index)).c_str(), 1);
    SamplingParams p;
    p.max_tokens = max_tokens;
    p.temperature = (float)o.temperature;
    p.seed = (uint64_t)o.seed;
    p.eos_token_ids = eos;
    p.ignore_eos = o.ignore_eos;
    engine.set_next_request_id(base);
    engine.synchronize();
    const auto t0 = std::chrono::steady_clock::now();
    const auto outputs = engine.generate(prompts, {p});
    const double wall = std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count();
    const Json* label = call.get("label");
    const GraphStats& g = engine.runner().graph_stats();
    char wall_text[40];
    std::snprintf(wall_text, sizeof wall_text, "%.9f", wall);
    records += std::string(index ? ", " : "") + "{\"label\": " + json_string(label ? label->text : std::to_string(index)) +
               ", \"request_id_base\": " + std::to_string(base) + ", \"input_token_ids\": " + ids_json(prompts) +
               ", \"output_token_ids\": " + ids_json(outputs) + ", \"reclaimed_pages_before_call\": " + std::to_string(dropped) +
               ", \"cache_isolated\": " + (prefix_caching ? "false" : "true") + ", \"cache_page_tokens\": " + std::to_string(engine.page_size()) +
               ", \"wall_s\": " + wall_text + ", \"graph_stats\": {\"eager\": " + std::to_string(g.eager) + ", \"captured\": " +
               std::to_string(g.captured) + ", \"replayed\": " + std::to_string(g.replayed) + ", \"evicted\": " + std::to_string(g.evicted) + "}}";
    base += prompts.size();
    prior.emplace_back(prompts, outputs);
  }
  records += "]";
  std::FILE* f = std::fopen(o.bench_call_results.c_str(), "wx");
  if (!f) throw Usage("bench calls: cannot create " + o.bench_call_results);
  std::fputs(records.c_str(), f);
  std::fclose(f);
  std::cout << "CALLS_FINISHED " << calls->items.size() << "\n";
  return 0;
}

int run(int argc, char** argv) {
  Options o = parse(argc, argv);
  for (const std::string& p : o.plugins) load_plugin(p);
  if (o.kind == "describe") {
    if (o.model_path.empty()) throw Usage("MODEL_PATH (or --model-path) is required");
    return describe(o);
  }
  EngineOptions eo;
  eo.model_dir = o.model_path;
  if (o.kind != "engine") throw Usage("--kind " + o.kind + ": this program is the engine; random-model is the Python launcher's");
  if (o.model_path.empty()) throw Usage("MODEL_PATH (or --model-path) is required");
  if (o.device != "cuda:0" && o.device != "cuda") throw Usage("device '" + o.device + "': this engine runs on cuda:0 only");
  if (o.dtype == "bfloat16" || o.dtype == "bf16") eo.dtype = "bf16";
  else if (o.dtype == "float32" || o.dtype == "f32") eo.dtype = "f32";
  else throw Usage("--dtype must be bfloat16 or float32");
  if (o.graphs != 0 && o.graphs != 1) throw Usage("--graphs must be 0 or 1");
  if (o.prefix_cache != 0 && o.prefix_cache != 1) throw Usage("--prefix-cache must be 0 or 1");
  if (o.temperature < 0) throw Usage("--temperature must not be negative");
  std::vector<Prepared> requests, warmup, primer;
  if (!o.bench_calls.empty()) {
  } else if (!o.bench_input.empty()) {
    requests = parse_prepared(o.bench_input);
  } else {
    requests.push_back({(int)o.max_tokens, parse_ids(o.prompt_ids), 0});
  }
  if (!o.bench_input.empty() && !o.bench_warmup_input.empty()) warmup = parse_prepared(o.bench_warmup_input);
  if (!warmup.empty() && !o.bench_graph_primer_input.empty()) primer = parse_prepared(o.bench_graph_primer_input);
  const std::vector<int32_t> eos = eos_ids(o.model_path);
  eo.lib_dir = o.lib_dir.empty() ? self_dir() : o.lib_dir;
  eo.num_pages = (int)o.num_blocks;
  eo.page_size = (int)o.page_size;
  eo.max_num_seqs = o.max_seqs > 0 ? (int)o.max_seqs
                                   : (int)std::max<size_t>({requests.size(), warmup.size(), primer.size(), o.bench_calls.empty() ? (size_t)1 : (size_t)8});
  eo.max_num_batched_tokens = (int)o.max_batched_tokens;
  eo.prefix_cache = o.prefix_cache == 1;
  eo.max_model_len = (int)o.max_model_len;
  eo.graphs = o.graphs == 1;
  if (!o.random_weights.empty()) {
    eo.random_weights = true;
    eo.random_seed = (uint64_t)to_int(o.random_weights, "--random-weights");
  }
  {
    // --family names: the model_type of every registered architecture.
    register_builtin_architectures();
    const auto types = model_types();
    std::string known;
    for (const auto& t : types) known += (known.empty() ? "" : ", ") + t.first;
    if (o.family.empty()) throw Usage("--family is required (one of: " + known + ")");
    auto it = types.find(o.family);
    if (it == types.end()) throw Usage("unknown --family " + o.family + " (one of: " + known + ")");
    const std::string architecture = model_spec_from_dir(o.model_path).architecture;
    if (architecture != it->second) throw Usage(o.model_path + " holds a " + architecture + ", not a " + o.family + " model");
  }
  eo.plugins = o.plugins;
  Engine engine(eo);
  if (!o.bench_calls.empty()) return run_calls(engine, o, eos);
  engine.record_step_times(!o.step_times.empty());
  std::FILE* trace = nullptr;
  if (!o.step_trace.empty()) {
    trace = std::fopen(o.step_trace.c_str(), "a");
    if (!trace) throw Usage("cannot open " + o.step_trace);
  }
  struct Served {
    std::vector<std::vector<int32_t>> outputs;
    double wall = 0;
    int64_t requests_with_reuse = 0, reused_blocks = 0;
  };
  auto serve = [&](const std::vector<Prepared>& reqs, long first_seed) {
    std::vector<SamplingParams> params;
    std::vector<std::vector<int32_t>> prompts;
    std::vector<int> arrivals;
    for (size_t i = 0; i < reqs.size(); ++i) {
      SamplingParams p;
      p.max_tokens = reqs[i].max_tokens;
      p.temperature = (float)o.temperature;
      p.seed = (uint64_t)(first_seed + (long)i);
      p.eos_token_ids = eos;
      p.ignore_eos = o.ignore_eos;
      params.push_back(p);
      prompts.push_back(reqs[i].ids);
      arrivals.push_back(reqs[i].arrival);
    }
    Served s;
    const int64_t before_requests = engine.cache().prefix_hit_requests(), before_blocks = engine.cache().prefix_hits();
    engine.synchronize();
    const auto t0 = std::chrono::steady_clock::now();
    s.outputs = engine.generate(prompts, params, arrivals, trace);
    s.wall = std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count();
    s.requests_with_reuse = engine.cache().prefix_hit_requests() - before_requests;
    s.reused_blocks = engine.cache().prefix_hits() - before_blocks;
    return s;
  };
  auto line = [](const char* tag, const std::vector<Prepared>& reqs, const Served& s, bool rate) {
    size_t n_out = 0, n_in = 0;
    for (const auto& out : s.outputs) n_out += out.size();
    for (const auto& r : reqs) n_in += r.ids.size();
    char buf[256];
    int n = std::snprintf(buf, sizeof buf, "%s batch=%zu prompt_tokens=%zu output_tokens=%zu wall_s=%.9f", tag, reqs.size(), n_in, n_out, s.wall);
    if (rate) std::snprintf(buf + n, sizeof buf - n, " tok_s=%.6f", (double)n_out / s.wall);
    return std::string(buf);
  };
  auto stats = [](const std::vector<Prepared>& reqs, const Served& s) {
    return "{\"admitted_requests\":" + std::to_string(reqs.size()) + ",\"requests_with_reuse\":" + std::to_string(s.requests_with_reuse) +
           ",\"reused_prefix_blocks\":" + std::to_string(s.reused_blocks);
  };
  if (!primer.empty()) {
    // An optional third workload, served first in the same engine, so that the recordings of the decode steps it
    // walks through exist before the warm-up (examples/support/engine_serving.rs:162-181).  Nothing is reported of it.
    setenv("VOSTI_LOGITS_OBSERVER_PHASE", "primer", 1);
    serve(primer, o.seed + (long)(requests.size() + warmup.size()));
  }
  if (!warmup.empty()) {
    // The reference serves a disjoint warm-up workload in the same engine before the measured one
    // (examples/support/engine_serving.rs:157-206) and reports both (engine_benchmark.rs:45-76).
    setenv("VOSTI_LOGITS_OBSERVER_PHASE", "warmup", 1);
    const Served w = serve(warmup, o.seed + (long)requests.size());
    std::cout << line("WARMUP", warmup, w, false) << "\n" << "WARMUP_CACHE_STATS " << stats(warmup, w) << "}\n";
  }
  if (!warmup.empty()) setenv("VOSTI_LOGITS_OBSERVER_PHASE", "measured", 1);
  const Served s = serve(requests, o.seed);
  if (trace) std::fclose(trace);
  if (!o.step_times.empty()) {
    std::ofstream f(o.step_times);
    char buf[96];
    for (const StepTime& t : engine.step_times()) {
      std::snprintf(buf, sizeof buf, "%d %d %d %.6f\n", t.rows, t.tokens, t.sampled, t.ms);
      f << buf;
    }
  }
  if (!o.output_tokens.empty()) {
    std::ofstream f(o.output_tokens);
    for (size_t i = 0; i < s.outputs.size(); ++i) f << i << "\t" << id_list(s.outputs[i], ",") << "\n";
  }
  if (!o.bench_input.empty()) {
    std::cout << line("BENCH", requests, s, true) << "\n";
    std::cout << "CACHE_STATS " << stats(requests, s) << ",\"preemptions\":" << engine.scheduler().preemptions() << "}\n";
  } else {
    std::cout << "MODEL_OUTPUT_TOKEN_IDS=[" << id_list(s.outputs[0], ", ") << "]\n";
  }
  if (o.graphs) {
    const GraphStats& g = engine.runner().graph_stats();
    std::cout << "GRAPH_STATS {\"eager\":" << g.eager << ",\"captured\":" << g.captured << ",\"replayed\":" << g.replayed
              << ",\"evicted\":" << g.evicted << "}\n";
  }
  std::cout.flush();
  return 0;
}

}  // namespace

int main(int argc, char** argv) {
  try {
    return run(argc, argv);
  } catch (const Usage& e) {
    std::cerr << "vosti_engine: " << e.what() << "\n";
    return 2;
  } catch (const std::exception& e) {
    std::cerr << "vosti_engine: " << e.what() << "\n";
    return 1;
  }
}
