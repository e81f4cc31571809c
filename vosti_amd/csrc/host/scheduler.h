// Continuous batching above the cache manager: admits requests, cuts prompts
// into portions under a token budget, decodes, finishes and frees.
//
// Policy, after the reference's planner (src/exec/cache_scheduler/planning.rs):
//   * requests wait in arrival order; ids are never reused (admission.rs:387-396)
//   * a step first takes the running requests in order: a decoding one
//     contributes its one pending token and is not limited by the token budget
//     (planning.rs:247-338); a request still inside its prompt contributes its
//     next portion
//   * then the head of the waiting queue is admitted while rows, running seats
//     and budget last (planning.rs:632-2625): the pages of its whole prompt are
//     taken at admission in the all-keys groups (planning.rs:992-998), leaving
//     one page of headroom for every running request whose next token opens a
//     new page (planning.rs:978-1001); a prompt that does not fit the rest of
//     the budget is cut at a page boundary (planning.rs:11-49), and when
//     nothing of it fits it stays at the head of the queue
//   * a row is sampled only if it ends its request's tokens (planning.rs:2080)
//   * a request ends on max_tokens or on one of its end tokens, which is still
//     emitted (request_state.rs:482-501), and its pages go back at once
//
// Where this scheduler decides for itself:
//   * a prompt cut into portions keeps its pages between the portions; the
//     reference parks it and finds its pages again through the prefix cache
//     (request_lifecycle.rs:187-316)
//   * a decoding request that needs a new page and finds none is left out of
//     the step; the others go on (the reference stops at the first one,
//     planning.rs:314-316)
//   * when no row at all can be scheduled although requests are running, the
//     youngest running request is preempted: its pages are freed and it returns
//     to the head of the waiting queue with its generated tokens as part of its
//     prompt, to be recomputed.  The reference makes no progress in that case
//     (cache_scheduler/mod.rs:8-12).  If a single request cannot fit the empty
//     pool, plan() reports OUT_OF_PAGES.
#pragma once
#include <cstdint>
#include <deque>
#include <unordered_map>
#include <unordered_set>
#include <vector>

#include "cache_manager.h"

namespace vosti {

enum AdmissionStatus : int {
  ACCEPTED = 0,
  DUPLICATE_REQUEST_ID = 1,
  EMPTY_PROMPT = 2,
  TOO_MANY_EOS_TOKEN_IDS = 3,
  ZERO_MAX_TOKENS = 4,
  HISTORY_CAPACITY_OVERFLOW = 5,
  EMPTY_EOS_TOKEN_IDS = 6,   // no end token although end tokens are not ignored (request_state.rs:207, engine.rs:2718-2720)
};

enum PlanStatus : int {
  PLAN_OK = 0,
  PLAN_IDLE = 1,          // nothing live
  PLAN_OUT_OF_PAGES = 2,  // a request cannot fit even the empty pool
  PLAN_STEP_PENDING = 3,  // the step planned before was neither committed nor given up
  PLAN_INTERNAL = 4,      // the cache manager refused a row for a reason other than pages: a fault of the engine
};

struct SchedulerConfig {
  int max_num_seqs;
  int max_num_batched_tokens;
  int max_model_len;   // prompt + generated tokens a request may reach
};

struct PlanRow {
  RequestId id;
  int start;      // position of the row's first token
  int n_tokens;
  int sample;     // 1: the row ends the request's tokens and a token is drawn
  int state_slot;
  int output_index;   // index of the token this row would emit
};

struct Emitted {
  RequestId id;
  int32_t token;
  int finished;
};

class Scheduler {
 public:
  Scheduler(CacheManager* cache, SchedulerConfig config);

  AdmissionStatus add_request(RequestId id, const int32_t* prompt, int n_prompt, int max_tokens,
                              const int32_t* eos, int n_eos, bool ignore_eos);

  // Decides the next step and takes its pages.  rows/tokens describe it:
  // tokens holds the rows' tokens back to back.
  PlanStatus plan(std::vector<PlanRow>& rows, std::vector<int32_t>& tokens);
  // The planned step ran; `sampled` has one token per sampled row, in row order.  False, and nothing
  // committed, if their number is not the number of sampled rows of the plan.
  bool commit(const int32_t* sampled, int n_sampled, std::vector<Emitted>& out);
  // The planned step did not run (a launch failed): the rows' tokens stay uncomputed, their pages stay
  // with their requests, and the next plan() decides again.
  void abort_step();
  int num_planned_samples() const;
  // Gives up a live request (waiting or running).
  bool abort(RequestId id);

  int num_waiting() const { return (int)waiting_.size(); }
  int num_running() const { return (int)running_.size(); }
  int64_t preemptions() const { return preemptions_; }
  bool is_live(RequestId id) const { return live_.count(id) != 0; }

 private:
  struct Request {
    std::vector<int32_t> tokens;   // prompt, then generated
    int n_prompt = 0;
    int generated = 0;
    int max_tokens = 0;
    std::vector<int32_t> eos;
    bool ignore_eos = false;
  };
  int try_rows(std::vector<PlanRow>& rows, std::vector<int32_t>& tokens);   // 1: rows, 0: none fit, -1: fault
  int chunk_for(int remaining, int available, bool first) const;
  int page_debt() const;

  CacheManager* cache_;
  SchedulerConfig config_;
  std::deque<RequestId> waiting_;
  std::vector<RequestId> running_;
  std::unordered_map<RequestId, Request> live_;
  std::unordered_set<RequestId> accepted_;   // every id ever taken
  std::vector<PlanRow> planned_;
  int64_t preemptions_ = 0;
};

}  // namespace vosti
