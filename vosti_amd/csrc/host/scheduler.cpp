#include "scheduler.h"

#include <algorithm>

namespace vosti {

Scheduler::Scheduler(CacheManager* cache, SchedulerConfig config) : cache_(cache), config_(config) {}

AdmissionStatus Scheduler::add_request(RequestId id, const int32_t* prompt, int n_prompt, int max_tokens,
                                       const int32_t* eos, int n_eos, bool ignore_eos) {
  if (accepted_.count(id)) return DUPLICATE_REQUEST_ID;
  if (n_prompt <= 0 || prompt == nullptr) return EMPTY_PROMPT;
  if (n_eos == 0 && !ignore_eos) return EMPTY_EOS_TOKEN_IDS;
  if (n_eos > 3 || n_eos < 0) return TOO_MANY_EOS_TOKEN_IDS;
  if (max_tokens <= 0) return ZERO_MAX_TOKENS;
  if ((int64_t)n_prompt + max_tokens > config_.max_model_len) return HISTORY_CAPACITY_OVERFLOW;
  Request r;
  r.tokens.assign(prompt, prompt + n_prompt);
  r.n_prompt = n_prompt;
  r.max_tokens = max_tokens;
  if (n_eos > 0) r.eos.assign(eos, eos + n_eos);
  r.ignore_eos = ignore_eos;
  accepted_.insert(id);
  live_.emplace(id, std::move(r));
  waiting_.push_back(id);
  return ACCEPTED;
}

int Scheduler::chunk_for(int remaining, int available, bool first) const {
  if (available <= 0) return 0;
  if (remaining <= available) return remaining;
  const int P = cache_->page_size();
  const int aligned = available / P * P;
  if (aligned > 0) return aligned;
  // A budget below one page: an unaligned portion, but only as the step's first
  // row, so that such a step always makes progress.
  return first ? available : 0;
}

int Scheduler::page_debt() const {
  int debt = 0;
  const int P = cache_->page_size();
  for (RequestId id : running_) {
    const int held = cache_->length(id) + cache_->pending(id);
    if (held % P == 0) debt += 1;
  }
  return debt;
}

int Scheduler::try_rows(std::vector<PlanRow>& rows, std::vector<int32_t>& tokens) {
  rows.clear();
  tokens.clear();
  int used = 0;
  const int budget = config_.max_num_batched_tokens;
  for (RequestId id : running_) {
    if ((int)rows.size() >= config_.max_num_seqs) break;
    Request& r = live_.at(id);
    const int computed = cache_->length(id);
    const int remaining = (int)r.tokens.size() - computed;
    const int n = remaining == 1 ? 1 : chunk_for(remaining, budget - used, rows.empty());
    if (n <= 0) continue;
    const Status st = cache_->extend(id, r.tokens.data() + computed, n);
    if (st == NO_PAGES) continue;            // left out of this step; the others go on
    if (st != OK) {                          // a step still pending, an unknown request: not a matter of pages
      for (const PlanRow& done : rows) cache_->abort_step(done.id);
      rows.clear();
      tokens.clear();
      return -1;
    }
    rows.push_back(PlanRow{id, computed, n, computed + n == (int)r.tokens.size() ? 1 : 0, cache_->state_slot(id),
                           r.generated});
    tokens.insert(tokens.end(), r.tokens.begin() + computed, r.tokens.begin() + computed + n);
    used += n;
  }
  while (!waiting_.empty() && (int)rows.size() < config_.max_num_seqs &&
         (int)running_.size() < config_.max_num_seqs) {
    const int available = budget - used;
    if (available <= 0) break;
    const RequestId id = waiting_.front();
    Request& r = live_.at(id);
    const int total = (int)r.tokens.size();
    int cached = 0;
    if (cache_->add_request(id, r.tokens.data(), total, &cached) != OK) break;
    const int remaining = total - cached;
    const int n = chunk_for(remaining, available, rows.empty());
    bool ok = n > 0;
    const int debt = page_debt();
    for (int g = 0; ok && g < cache_->num_groups(); ++g) {
      const int more = cache_->window(g) == 0 ? remaining : n;
      const int head = cache_->window(g) == 0 ? debt : 0;
      if (cache_->pages_needed(id, g, more) + head > cache_->available_pages(g)) ok = false;
    }
    ok = ok && cache_->reserve(id, total) == OK && cache_->extend(id, r.tokens.data() + cached, n) == OK;
    if (!ok) {
      cache_->finish(id);
      break;
    }
    waiting_.pop_front();
    running_.push_back(id);
    rows.push_back(PlanRow{id, cached, n, cached + n == total ? 1 : 0, cache_->state_slot(id), r.generated});
    tokens.insert(tokens.end(), r.tokens.begin() + cached, r.tokens.begin() + cached + n);
    used += n;
  }
  return rows.empty() ? 0 : 1;
}

PlanStatus Scheduler::plan(std::vector<PlanRow>& rows, std::vector<int32_t>& tokens) {
  if (!planned_.empty()) {
    rows.clear();
    tokens.clear();
    return PLAN_STEP_PENDING;
  }
  if (live_.empty()) {
    rows.clear();
    tokens.clear();
    return PLAN_IDLE;
  }
  for (;;) {
    const int got = try_rows(rows, tokens);
    if (got < 0) return PLAN_INTERNAL;
    if (got > 0) {
      planned_ = rows;
      return PLAN_OK;
    }
    if (running_.size() < 2) return PLAN_OUT_OF_PAGES;
    const RequestId victim = running_.back();
    running_.pop_back();
    cache_->finish(victim);
    waiting_.push_front(victim);
    preemptions_ += 1;
  }
}

int Scheduler::num_planned_samples() const {
  int n = 0;
  for (const PlanRow& row : planned_)
    if (row.sample && live_.count(row.id)) n += 1;
  return n;
}

void Scheduler::abort_step() {
  for (const PlanRow& row : planned_)
    if (live_.count(row.id)) cache_->abort_step(row.id);
  planned_.clear();
}

bool Scheduler::commit(const int32_t* sampled, int n_sampled, std::vector<Emitted>& out) {
  out.clear();
  if (n_sampled != num_planned_samples() || (n_sampled > 0 && sampled == nullptr)) return false;
  int k = 0;
  for (const PlanRow& row : planned_) {
    auto it = live_.find(row.id);
    if (it == live_.end()) continue;
    cache_->commit(row.id);
    if (!row.sample) continue;
    Request& r = it->second;
    const int32_t tok = sampled[k++];
    r.tokens.push_back(tok);
    r.generated += 1;
    bool finished = r.generated >= r.max_tokens;
    if (!r.ignore_eos && std::find(r.eos.begin(), r.eos.end(), tok) != r.eos.end()) finished = true;
    out.push_back(Emitted{row.id, tok, finished ? 1 : 0});
    if (finished) {
      cache_->finish(row.id);
      running_.erase(std::find(running_.begin(), running_.end(), row.id));
      live_.erase(it);
    }
  }
  planned_.clear();
  return true;
}

bool Scheduler::abort(RequestId id) {
  auto it = live_.find(id);
  if (it == live_.end()) return false;
  auto w = std::find(waiting_.begin(), waiting_.end(), id);
  if (w != waiting_.end()) waiting_.erase(w);
  auto r = std::find(running_.begin(), running_.end(), id);
  if (r != running_.end()) {
    running_.erase(r);
    cache_->finish(id);
  }
  planned_.erase(std::remove_if(planned_.begin(), planned_.end(), [id](const PlanRow& p) { return p.id == id; }),
                 planned_.end());
  live_.erase(it);
  return true;
}

}  // namespace vosti
