// Requests, the per-step plan, and the scheduler that writes it.
//
// Every engine step the scheduler (1) gives each running request its next tokens: one token
// when it is decoding, a portion of its prompt under the step's token budget when it is still
// prefilling, taking pages as needed and preempting the newest admitted request when a pool
// is empty; (2) admits waiting requests in policy order while there is room, budget and
// memory (reference: mercury/scheduler.py:122-179, which admits whole prompts only; the three
// policies, and what each does when the head of the queue does not fit, are the reference's:
// mercury/scheduler.py:103-120, :155-160).
//
// When pages run out the newest admitted request loses everything it holds and goes back to
// the waiting queue at its original arrival time; it later starts over with prompt plus
// generated tokens as its prompt (reference: mercury/scheduler.py:91-101).
#pragma once

#include <cmath>
#include <cstdint>
#include <limits>
#include <memory>
#include <string>
#include <vector>

#include "cache_manager.h"
#include "hashing.h"

namespace mercury {

enum class RequestState { WAITING, RUNNING, FINISHED, ABORTED };
const char* state_name(RequestState s);

// temperature <= 0 is greedy; top_p < 1 keeps the nucleus; `seed`, when set, replaces the
// engine's seed for this request's random stream (the reference stores a seed and never
// reads it, mercury/request.py:14-23).
struct SamplingParams {
  double temperature = 0.0;
  double top_p = 1.0;
  bool ignore_eos = false;
  bool has_seed = false;
  int64_t seed = 0;
  bool greedy() const { return temperature <= 0.0; }
};

constexpr double kNever = std::numeric_limits<double>::quiet_NaN();

struct Request {
  std::string rid;
  std::vector<int32_t> tokens;      // prompt followed by the generated tokens
  int prompt_len = 0;
  int max_tokens = 0;
  double arrival = 0.0;
  uint64_t order = 0;               // submission order, the tie-break among equal arrivals
  std::vector<PageHash> chain;      // hashes of the full pages of `tokens` known so far
  SamplingParams params;
  std::string session_id;
  bool has_session = false;

  int num_computed = 0;             // tokens whose keys and values are in the cache
  int num_cached = 0;               // of those, how many admission found already cached
  RequestState state = RequestState::WAITING;
  double admitted_at = kNever, last_admitted_at = kNever, first_token_at = kNever,
         finished_at = kNever;
  int preemptions = 0;
  int64_t recomputed_tokens = 0;
  std::string finish_reason;

  int seq_len() const { return (int)tokens.size(); }
  int num_out() const { return (int)tokens.size() - prompt_len; }
  int remaining() const { return seq_len() - num_computed; }   // tokens to run before sampling
  bool running() const { return state == RequestState::RUNNING; }
  bool done() const { return state == RequestState::FINISHED || state == RequestState::ABORTED; }
  void append(int32_t token) { tokens.push_back(token); }
};

using RequestPtr = std::shared_ptr<Request>;

// Tokens [start, start + count) of a request run this step; `emits` when they complete the
// sequence, so that the step's last logits give the request's next token.
struct Work {
  RequestPtr request;
  int start = 0, count = 0;
  bool emits = false;
  bool decode() const { return count == 1 && emits && start >= request->prompt_len; }
};

struct Plan {
  std::vector<Work> work;
  std::vector<RequestPtr> preempted, admitted;
  double sched_seconds = 0.0;
  // The next plan is expected to be this one a token further: every request decodes and none
  // reaches its length limit with this step's token, and nobody waits for a place that is
  // free.  (A stop token may still prove it wrong.)  An executor may start the next step's
  // work early on the strength of it.
  bool steady = false;

  int num_decode() const;
  int num_prefill() const { return (int)work.size() - num_decode(); }
  int num_prefill_tokens() const;
};

enum class Policy { FCFS, LPM, LPM_AGING };
Policy parse_policy(const std::string& name);

struct SchedulerOptions {
  Policy policy = Policy::FCFS;
  int max_running = 64;
  int prefill_budget = 8192;
  double aging_tokens_per_s = 2000.0;
  double max_wait_s = 5.0;
  int scan_limit = 128;
};

class Scheduler {
 public:
  struct Stats {
    int64_t steps = 0, preemptions = 0, admissions = 0, max_waiting = 0, scan_limit_exceeded = 0,
            scored_requests = 0;
    double sched_seconds = 0.0;
  };

  Scheduler(std::shared_ptr<CacheManager> manager, std::shared_ptr<PageHasher> hasher,
            SchedulerOptions options);

  const SchedulerOptions& options() const { return options_; }
  SchedulerOptions& mutable_options() { return options_; }
  const std::vector<RequestPtr>& waiting() const { return waiting_; }
  const std::vector<RequestPtr>& running() const { return running_; }
  const Stats& stats() const { return stats_; }
  bool has_work() const { return !waiting_.empty() || !running_.empty(); }

  void add(const RequestPtr& r);                 // into the waiting queue, by arrival
  RequestPtr abort(const std::string& rid);      // null when the request is unknown
  void drop(const RequestPtr& r);                // finished: everything it holds goes back
  Plan schedule(double now);
  double score(const Request& r, double now) const;

 private:
  void release(const Request& r);
  void preempt(const RequestPtr& r);
  void continue_running(Plan& plan, int& budget);
  void admit_waiting(Plan& plan, int& budget, double now);

  std::shared_ptr<CacheManager> manager_;
  std::shared_ptr<PageHasher> hasher_;
  SchedulerOptions options_;
  std::vector<RequestPtr> waiting_, running_;
  Stats stats_;
};

}  // namespace mercury
