// The engine: requests in, tokens out.
//
// One step is plan -> forward -> sample -> commit, as in the reference (src/exec/engine.rs:2795, 2862, 3258,
// 3427; docs/architecture.md:99-109).  The scheduler decides the rows and takes their pages, the step
// function runs them and returns logits at the rows that end a request's tokens, the sampler draws one
// token per such row on the GPU, and one readback per step brings the tokens to the host, where the
// scheduler appends them and retires finished requests.
#pragma once
#include <cstdio>
#include <map>
#include <memory>
#include <string>
#include <vector>

#include "../host/scheduler.h"
#include "observe.h"
#include "runner.h"

namespace vosti {

// The reference samples greedily only (python/vosti_kernels/kernels.py:1088-1104) and stops on max_tokens
// or on one of up to three end tokens unless they are ignored (src/exec/request_state.rs:97-187, 418-446).
// Temperature sampling is this engine's own: the uniform number that picks output token i of a request is a
// function of (the request's seed, i) alone, so what a request generates does not depend on its companions
// in a batch or on how its work was cut.
struct SamplingParams {
  int max_tokens = 8;
  float temperature = 0.f;       // 0: greedy
  uint64_t seed = 0;
  std::vector<int32_t> eos_token_ids;
  bool ignore_eos = false;
};

// The uniform number in [0, 1) for output token `output_index` of a request with `seed`: 24 bits.
float uniform_for(uint64_t seed, uint64_t output_index);

struct EngineOptions {
  std::string model_dir, lib_dir;
  std::string dtype = "bf16";    // "bf16" or "f32"
  int num_pages = 32;            // the reference's VOSTI_NUM_BLOCKS (examples/support/engine_setup.rs:57-69)
  int page_size = 64;
  int max_num_seqs = 8;          // VOSTI_MAX_SEQS
  int max_num_batched_tokens = 4096;   // VOSTI_MAX_BATCHED_TOKENS
  bool prefix_cache = true;
  int max_model_len = 0;         // 0: the model's positions
  bool graphs = false;           // VOSTI_CUDA_GRAPH (engine_setup.rs:79-81)
  bool random_weights = false;   // draw the weights from random_seed on the GPU; the folder needs config.json only
  uint64_t random_seed = 0;
  std::vector<std::string> plugins;    // shared libraries with part kinds and architectures of their own (load_plugin)
};

// Why this engine cannot run the model in the folder, or "" if it can: an architecture that is not registered,
// or a part kind that its description names and no registered part has.  Configuration errors are thrown.
std::string why_unsupported(const std::string& model_dir);

// What one engine step took, for measurements.
struct StepTime {
  int rows = 0, tokens = 0, sampled = 0;
  double ms = 0.0;               // plan, forward, sample, readback and commit, by the host's clock
};

class Engine {
 public:
  explicit Engine(const EngineOptions& opt);
  ~Engine();

  RequestId add_request(const std::vector<int32_t>& prompt, const SamplingParams& params);
  bool has_unfinished() const { return !params_.empty(); }
  // One engine step.  Returns (request, emitted token) for the requests that emitted one.
  std::vector<std::pair<RequestId, int32_t>> step();
  // Generates for every prompt; arrival_steps[i] delays prompt i until that engine step (the reference's
  // prepared-request file has the same column: examples/support/engine_benchmark.rs:89-165).  trace: a file
  // that gets one JSON line per step (engine_benchmark.rs:212-220, 273-317).
  std::vector<std::vector<int32_t>> generate(const std::vector<std::vector<int32_t>>& prompts, const std::vector<SamplingParams>& params,
                                             const std::vector<int>& arrival_steps = {}, std::FILE* trace = nullptr);
  void synchronize();

  CacheManager& cache() { return pool_->manager(); }
  Scheduler& scheduler() { return *scheduler_; }
  ModelRunner& runner() { return *runner_; }
  DecoderModel& model() { return *model_; }
  const std::vector<RequestId>& last_scheduled() const { return last_scheduled_; }
  // Requests added from now on get ids from `id` on (never below what was given out already): the reference's
  // drivers give every workload of one engine a base of its own (examples/support/engine_calls.rs:70-118).
  void set_next_request_id(RequestId id) { next_id_ = std::max(next_id_, id); }
  int page_size() const { return pool_->page_size; }
  void record_step_times(bool on) { record_times_ = on; }
  const std::vector<StepTime>& step_times() const { return step_times_; }

 private:
  std::vector<int32_t> forward_and_sample(const std::vector<PlanRow>& rows, const std::vector<int32_t>& tokens);

  std::unique_ptr<Kernels> kernels_;
  std::unique_ptr<DecoderModel> model_;
  std::unique_ptr<CachePool> pool_;
  std::unique_ptr<ModelRunner> runner_;
  std::unique_ptr<Scheduler> scheduler_;
  int max_model_len_ = 0;
  // Fixed-size per-request state, by state slot: the sampler's.
  std::vector<float> slot_temperature_;
  std::vector<uint64_t> slot_seed_;
  std::vector<int64_t> slot_owner_;
  std::map<RequestId, SamplingParams> params_;
  RequestId next_id_ = 0;
  int64_t steps_ = 0;
  std::vector<RequestId> last_scheduled_;
  bool record_times_ = false;
  std::vector<StepTime> step_times_;
  // VOSTI_LOGITS_DIGEST / VOSTI_LOGITS_OBSERVER_DIR: hashes or copies of every sampled logits row, to compare runs
  // that batch differently (python/vosti_kernels/kernels.py:1020-1033).
  LogitsObserver observer_;
  std::vector<float> observed_;
  // The sampler's buffers: temperatures and uniform numbers up, token ids down.
  float* sample_in_ = nullptr;        // pinned [2, rows]
  int32_t* sample_out_ = nullptr;     // pinned [rows]
  std::unique_ptr<DeviceBuffer> sample_dev_;
  int sample_rows_ = 0;
  size_t sample_stride() const { return ((size_t)sample_rows_ * 4 + 255) & ~(size_t)255; }   // bytes between the device arrays
};

}  // namespace vosti
