// The engine's bookkeeping for one step after another: submission checks, the scheduler's
// plan, what the executed plan means for every request (progress, pages that became
// shareable, pages a window passed, the sampled token, finishing), and the step log
// (reference: mercury/engine.py:104-252, mercury/metrics.py:7-112).
//
// The core emits nothing itself: `advance` and `abort` return the events that the step
// produced, and the caller (the Python engine, which owns the threads and the per-request
// sinks) delivers them.
#pragma once

#include <deque>
#include <map>
#include <set>
#include <string>
#include <utility>
#include <vector>

#include "scheduler.h"

namespace mercury {

// kind: "token" (token, index), "done" (finish_reason: "length" | "stop" | "abort"),
// "preempted", or "error" (message).
struct Event {
  std::string rid, kind;
  int token = -1;
  int index = 0;
  std::string finish_reason, message;
  double t = 0.0;
};

struct StepRecord {
  double t = 0;
  int num_prefill = 0, num_decode = 0, prefill_tokens = 0;
  double sched_s = 0, prepare_s = 0, forward_s = 0, device_s = 0, step_s = 0;
  int waiting = 0, running = 0, free_blocks = 0, preempted = 0;
};

struct RequestRecord {
  std::string rid, session_id, finish_reason, state;
  bool has_session = false;
  double arrival = 0, admitted_at = kNever, first_token_at = kNever, finished_at = kNever;
  int prompt_tokens = 0, output_tokens = 0, cached_tokens = 0, preemptions = 0;
  int64_t recomputed_tokens = 0;
};

RequestRecord record_of(const Request& r);

class EngineCore {
 public:
  EngineCore(std::shared_ptr<CacheManager> manager, std::shared_ptr<PageHasher> hasher,
             SchedulerOptions options, int max_model_len, std::vector<int> eos_ids,
             size_t max_step_records, size_t max_request_records);

  CacheManager& manager() { return *manager_; }
  Scheduler& scheduler() { return scheduler_; }
  const std::set<int>& eos_ids() const { return eos_ids_; }
  void set_eos_ids(const std::vector<int>& ids) { eos_ids_ = std::set<int>(ids.begin(), ids.end()); }

  // Why a submission cannot be taken, or "" when it can: an empty prompt, or a prompt and
  // token limit beyond what one request may ever hold.
  std::string refusal(size_t prompt_len, int max_tokens) const;
  RequestPtr make_request(const std::string& rid, std::vector<int32_t> prompt, int max_tokens,
                          double arrival, const SamplingParams& params, const std::string* session);
  void count_rejected() { ++counters_["rejected_requests"]; }

  void add(const RequestPtr& r) { scheduler_.add(r); }
  // The aborted request's closing event, or nothing when the request is unknown.
  std::vector<Event> abort(const std::string& rid, double now);
  // The step's plan, and a "preempted" event for every request that lost its place.
  Plan schedule(double now, std::vector<Event>& events);
  // The plan has run: tokens[i] is the token sampled for work[i], or -1 when that work did
  // not complete its sequence.
  std::vector<Event> advance(const Plan& plan, const std::vector<int>& tokens, double now);
  void count_idle() { ++counters_["idle_steps"]; }
  void log_step(const Plan& plan, double now, double prepare_s, double forward_s, double device_s,
                double step_s);

  const std::deque<StepRecord>& steps() const { return steps_; }
  const std::map<std::string, int64_t>& counters() const { return counters_; }
  std::vector<std::pair<std::string, double>> summary() const;
  std::vector<RequestRecord> drain_finished();

 private:
  void finish(const RequestPtr& r, const char* reason, double now, std::vector<Event>& events);

  std::shared_ptr<CacheManager> manager_;
  std::shared_ptr<PageHasher> hasher_;
  Scheduler scheduler_;
  int max_model_len_;
  std::set<int> eos_ids_;
  size_t max_step_records_, max_request_records_;
  std::deque<StepRecord> steps_;
  std::deque<RequestRecord> finished_;
  std::map<std::string, int64_t> counters_;
  uint64_t submitted_ = 0;
};

}  // namespace mercury
