#include "engine.h"

#include <algorithm>
#include <chrono>
#include <numeric>

namespace vosti {

static uint64_t mix64(uint64_t z) {
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}

float uniform_for(uint64_t seed, uint64_t output_index) {
  const uint64_t z = mix64(mix64(seed) ^ (output_index * 0x9E3779B97F4A7C15ull));
  return (float)(z >> 40) * (1.0f / 16777216.0f);
}

static const char* ADMISSION[] = {"Accepted", "DuplicateRequestId", "EmptyPrompt", "TooManyEosTokenIds", "ZeroMaxTokens",
                                  "HistoryCapacityOverflow", "EmptyEosTokenIds"};

std::string why_unsupported(const std::string& model_dir) {
  register_builtin_architectures();
  register_standard_parts();
  const std::string path = model_dir + "/config.json";
  if (!file_exists(path)) throw ConfigError(path + " is missing");
  Json raw;
  try {
    raw = Json::parse(read_text_file(path));
  } catch (const JsonError& e) {
    throw ConfigError(path + ": " + e.what());
  }
  if (!architecture_known(raw)) {
    const Json* archs = raw.get("architectures");
    const std::string name = (archs && archs->kind == Json::Array && !archs->items.empty()) ? archs->items[0].text : "";
    return "architecture '" + name + "' is not registered in the native engine";
  }
  const std::string missing = missing_part(model_spec_from_config(raw));
  return missing.empty() ? "" : "the native engine has no " + missing;
}

Engine::Engine(const EngineOptions& opt) {
  register_builtin_architectures();
  register_standard_parts();
  for (const std::string& p : opt.plugins) load_plugin(p);
  int devices = 0;
  hip_check(hipGetDeviceCount(&devices), "looking for a GPU");
  if (devices < 1) throw EngineError("no GPU: this engine has no CPU path");
  hip_check(hipSetDevice(0), "choosing the GPU");
  ModelSpec spec = model_spec_from_dir(opt.model_dir);
  kernels_ = std::make_unique<Kernels>(opt.lib_dir, opt.dtype);
  model_ = std::make_unique<DecoderModel>(std::move(spec), *kernels_);
  if (opt.random_weights) {
    model_->random_weights(opt.random_seed);
  } else {
    Checkpoint ckpt(opt.model_dir);
    model_->load_weights(ckpt);
  }
  if (opt.max_num_seqs <= 0 || opt.max_num_batched_tokens <= 0) throw EngineError("max_num_seqs and max_num_batched_tokens must be positive");
  // One state slot per request that can be alive: those running plus the one being admitted.
  const int slots = opt.max_num_seqs + 1;
  pool_ = std::make_unique<CachePool>(*model_, opt.page_size, opt.num_pages, slots, opt.prefix_cache);
  runner_ = std::make_unique<ModelRunner>(*model_, *pool_, opt.graphs);
  const int positions = (int)model_->spec().max_positions;
  max_model_len_ = std::min(opt.max_model_len > 0 ? opt.max_model_len : positions, positions);
  scheduler_ = std::make_unique<Scheduler>(&pool_->manager(), SchedulerConfig{opt.max_num_seqs, opt.max_num_batched_tokens, max_model_len_});
  slot_temperature_.assign(slots, 0.f);
  slot_seed_.assign(slots, 0);
  slot_owner_.assign(slots, -1);
  sample_rows_ = opt.max_num_seqs;
  hip_check(hipHostMalloc(reinterpret_cast<void**>(&sample_in_), 2 * sample_rows_ * sizeof(float), hipHostMallocDefault), "pinned allocation");
  hip_check(hipHostMalloc(reinterpret_cast<void**>(&sample_out_), sample_rows_ * sizeof(int32_t), hipHostMallocDefault), "pinned allocation");
  // [temperatures | uniform numbers | token ids | the sampler's scratch]
  sample_dev_ = std::make_unique<DeviceBuffer>(3 * sample_stride() + (size_t)kernels_->sample_scratch_words(sample_rows_) * 4);
}

Engine::~Engine() {
  if (kernels_) (void)hipStreamSynchronize(kernels_->stream);
  runner_.reset();
  if (sample_in_) (void)hipHostFree(sample_in_);
  if (sample_out_) (void)hipHostFree(sample_out_);
}

void Engine::synchronize() { hip_check(hipStreamSynchronize(kernels_->stream), "waiting for the stream"); }

RequestId Engine::add_request(const std::vector<int32_t>& prompt, const SamplingParams& params) {
  if (params.max_tokens <= 0) throw EngineError("max_tokens must be positive");
  if (params.temperature < 0) throw EngineError("temperature must not be negative");
  if (params.eos_token_ids.size() > 3) throw EngineError("at most three end tokens");
  const RequestId id = next_id_++;
  const int64_t vocab = model_->spec().vocab_size;
  for (int32_t t : prompt)
    if (t < 0 || t >= vocab) throw EngineError("prompt token outside [0, " + std::to_string(vocab) + ")");
  // A request without end tokens runs to max_tokens.
  const bool ignore = params.ignore_eos || params.eos_token_ids.empty();
  const AdmissionStatus st = scheduler_->add_request(id, prompt.data(), (int)prompt.size(), params.max_tokens, params.eos_token_ids.data(),
                                                     (int)params.eos_token_ids.size(), ignore);
  if (st != ACCEPTED) throw EngineError("request " + std::to_string(id) + " refused: " + ADMISSION[st]);
  params_[id] = params;
  return id;
}

std::vector<std::pair<RequestId, int32_t>> Engine::step() {
  const auto t0 = std::chrono::steady_clock::now();
  std::vector<PlanRow> rows;
  std::vector<int32_t> tokens;
  const PlanStatus st = scheduler_->plan(rows, tokens);
  if (st == PLAN_OUT_OF_PAGES) throw EngineError("a request needs more cache pages than the pool has, even alone");
  if (st == PLAN_STEP_PENDING) throw EngineError("plan() before the step planned last was committed or given up");
  if (st == PLAN_INTERNAL) throw EngineError("the cache manager refused a planned row for a reason other than pages");
  last_scheduled_.clear();
  for (const PlanRow& r : rows) last_scheduled_.push_back(r.id);
  std::vector<std::pair<RequestId, int32_t>> out;
  if (st == PLAN_IDLE || rows.empty()) return out;
  std::vector<int32_t> sampled;
  try {
    sampled = forward_and_sample(rows, tokens);
  } catch (...) {
    // Nothing of the step counts: the rows' tokens stay uncomputed, their pages stay with their requests,
    // and the next plan() decides again.
    scheduler_->abort_step();
    throw;
  }
  std::vector<Emitted> emitted;
  if (!scheduler_->commit(sampled.data(), (int)sampled.size(), emitted))
    throw EngineError("the scheduler refused " + std::to_string(sampled.size()) + " sampled tokens for a plan with " +
                      std::to_string(scheduler_->num_planned_samples()) + " sampled rows");
  ++steps_;
  if (record_times_) {
    StepTime t;
    t.rows = (int)rows.size();
    t.tokens = (int)tokens.size();
    t.sampled = (int)sampled.size();
    if (sampled.empty()) synchronize();          // a step without a readback has not waited for the GPU yet
    t.ms = std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - t0).count();
    step_times_.push_back(t);
  }
  for (const Emitted& e : emitted) {
    out.emplace_back(e.id, e.token);
    if (e.finished) params_.erase(e.id);
  }
  return out;
}

// Runs the planned rows and draws one token per sampled row (one readback).
std::vector<int32_t> Engine::forward_and_sample(const std::vector<PlanRow>& rows, const std::vector<int32_t>& tokens) {
  std::vector<StepEntry> entries;
  std::vector<const PlanRow*> sampling;
  size_t at = 0;
  for (const PlanRow& r : rows) {
    StepEntry e;
    e.id = r.id;
    e.tokens.assign(tokens.begin() + at, tokens.begin() + at + r.n_tokens);
    at += r.n_tokens;
    if (r.sample) {
      e.want.push_back(r.n_tokens - 1);
      sampling.push_back(&r);
    }
    entries.push_back(std::move(e));
  }
  Tensor logits = runner_->run(entries);
  std::vector<int32_t> sampled;
  const int R = (int)sampling.size();
  if (R == 0) return sampled;
  if (R > sample_rows_) throw EngineError("more sampled rows than the engine was made for");
  if (observer_.active()) {
    const Tensor f = kernels_->to_f32(logits);
    observed_.resize((size_t)f.numel());
    hip_check(hipMemcpyAsync(observed_.data(), f.data, f.bytes(), hipMemcpyDeviceToHost, kernels_->stream), "logits readback");
    hip_check(hipStreamSynchronize(kernels_->stream), "logits readback");
    std::vector<int> places;
    for (size_t i = 0; i < rows.size(); ++i)
      if (rows[i].sample) places.push_back((int)i);
    observer_.rows(observed_.data(), logits.dim(1), places, steps_, dtype_name(kernels_->dtype()));
  }
  bool any_temperature = false;
  for (int i = 0; i < R; ++i) {
    const PlanRow& r = *sampling[i];
    // The slot holds the request's sampler state.  A request gets its slot at admission, inside plan(), so
    // the state is written when the request's first sampled row shows up.
    if (slot_owner_.at(r.state_slot) != (int64_t)r.id) {
      const SamplingParams& p = params_.at(r.id);
      slot_owner_[r.state_slot] = (int64_t)r.id;
      slot_temperature_[r.state_slot] = p.temperature;
      slot_seed_[r.state_slot] = p.seed;
    }
    sample_in_[i] = slot_temperature_[r.state_slot];
    sample_in_[R + i] = uniform_for(slot_seed_[r.state_slot], (uint64_t)r.output_index);
    any_temperature = any_temperature || sample_in_[i] > 0.f;
  }
  hipStream_t st = kernels_->stream;
  char* dev = static_cast<char*>(sample_dev_->data());
  Tensor temps, unis, ids, scratch;
  temps.dtype = unis.dtype = DType::F32;
  ids.dtype = scratch.dtype = DType::I32;
  temps.shape = unis.shape = ids.shape = {R};
  temps.data = dev;
  unis.data = dev + sample_stride();
  ids.data = dev + 2 * sample_stride();
  scratch.data = dev + 3 * sample_stride();
  scratch.shape = {kernels_->sample_scratch_words(sample_rows_)};
  if (any_temperature) {
    hip_check(hipMemcpyAsync(temps.data, sample_in_, (size_t)R * sizeof(float), hipMemcpyHostToDevice, st), "sampler upload");
    hip_check(hipMemcpyAsync(unis.data, sample_in_ + R, (size_t)R * sizeof(float), hipMemcpyHostToDevice, st), "sampler upload");
  }
  kernels_->sample(ids, logits, any_temperature ? &temps : nullptr, any_temperature ? &unis : nullptr, scratch);
  hip_check(hipMemcpyAsync(sample_out_, ids.data, (size_t)R * sizeof(int32_t), hipMemcpyDeviceToHost, st), "token readback");
  hip_check(hipStreamSynchronize(st), "the step");        // the step's one synchronisation
  sampled.assign(sample_out_, sample_out_ + R);
  return sampled;
}

std::vector<std::vector<int32_t>> Engine::generate(const std::vector<std::vector<int32_t>>& prompts, const std::vector<SamplingParams>& params,
                                                   const std::vector<int>& arrival_steps, std::FILE* trace) {
  if (params.size() != prompts.size() && params.size() != 1) throw EngineError("one set of sampling parameters, or one per prompt");
  if (!arrival_steps.empty() && arrival_steps.size() != prompts.size()) throw EngineError("one arrival step per prompt");
  std::vector<size_t> pending(prompts.size());
  std::iota(pending.begin(), pending.end(), 0);
  auto arrival = [&](size_t i) { return arrival_steps.empty() ? 0 : arrival_steps[i]; };
  std::stable_sort(pending.begin(), pending.end(), [&](size_t a, size_t b) { return arrival(a) < arrival(b); });
  std::map<RequestId, size_t> index;
  std::vector<std::vector<int32_t>> outputs(prompts.size());
  size_t next = 0;
  for (int step_no = 0; next < pending.size() || has_unfinished(); ++step_no) {
    std::vector<size_t> arrived;
    while (next < pending.size() && arrival(pending[next]) <= step_no) {
      const size_t i = pending[next++];
      index[add_request(prompts[i], params.size() == 1 ? params[0] : params[i])] = i;
      arrived.push_back(i);
    }
    const auto emitted = step();
    for (const auto& e : emitted) {
      auto it = index.find(e.first);
      if (it != index.end()) outputs[it->second].push_back(e.second);
    }
    if (trace) {
      std::string line = "{\"step\": " + std::to_string(step_no) + ", \"arrived\": [";
      for (size_t i = 0; i < arrived.size(); ++i) line += (i ? ", " : "") + std::to_string(arrived[i]);
      line += "], \"scheduled\": [";
      for (size_t i = 0; i < last_scheduled_.size(); ++i) line += (i ? ", " : "") + std::to_string(last_scheduled_[i]);
      line += "], \"emitted\": {";
      for (size_t i = 0; i < emitted.size(); ++i) {
        auto it = index.find(emitted[i].first);
        const uint64_t shown = it != index.end() ? (uint64_t)it->second : (uint64_t)emitted[i].first;
        line += (i ? ", " : "") + ("\"" + std::to_string(shown) + "\": ") + std::to_string(emitted[i].second);
      }
      line += "}, \"cached_prefix_pages\": " + std::to_string(cache().prefix_hits()) + "}\n";
      std::fputs(line.c_str(), trace);
    }
  }
  return outputs;
}

}  // namespace vosti
