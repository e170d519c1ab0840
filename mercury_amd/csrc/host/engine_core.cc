#include "engine_core.h"

#include <algorithm>
#include <numeric>

namespace mercury {

RequestRecord record_of(const Request& r) {
  RequestRecord out;
  out.rid = r.rid;
  out.session_id = r.session_id;
  out.has_session = r.has_session;
  out.finish_reason = r.finish_reason;
  out.state = state_name(r.state);
  out.arrival = r.arrival;
  out.admitted_at = r.admitted_at;
  out.first_token_at = r.first_token_at;
  out.finished_at = r.finished_at;
  out.prompt_tokens = r.prompt_len;
  out.output_tokens = r.num_out();
  out.cached_tokens = r.num_cached;
  out.preemptions = r.preemptions;
  out.recomputed_tokens = r.recomputed_tokens;
  return out;
}

EngineCore::EngineCore(std::shared_ptr<CacheManager> manager, std::shared_ptr<PageHasher> hasher,
                       SchedulerOptions options, int max_model_len, std::vector<int> eos_ids,
                       size_t max_step_records, size_t max_request_records)
    : manager_(manager), hasher_(hasher), scheduler_(manager, hasher, options),
      max_model_len_(max_model_len), eos_ids_(eos_ids.begin(), eos_ids.end()),
      max_step_records_(max_step_records), max_request_records_(max_request_records) {
  for (const char* name : {"steps", "idle_steps", "prefill_requests", "prefill_tokens",
                           "decode_tokens", "finished_requests", "aborted_requests",
                           "rejected_requests", "preemptions"}) {
    counters_[name] = 0;
  }
}

std::string EngineCore::refusal(size_t prompt_len, int max_tokens) const {
  if (prompt_len == 0) return "prompt must contain at least one token";
  const long long ceiling = std::min<long long>(max_model_len_, manager_->capacity_tokens());
  if ((long long)prompt_len + max_tokens > ceiling) {
    return "prompt (" + std::to_string(prompt_len) + ") + max_tokens (" +
           std::to_string(max_tokens) + ") exceeds the " + std::to_string(ceiling) +
           "-token ceiling of this engine";
  }
  return "";
}

RequestPtr EngineCore::make_request(const std::string& rid, std::vector<int32_t> prompt,
                                    int max_tokens, double arrival, const SamplingParams& params,
                                    const std::string* session) {
  auto r = std::make_shared<Request>();
  r->rid = rid;
  r->prompt_len = (int)prompt.size();
  r->tokens = std::move(prompt);
  r->max_tokens = max_tokens;
  r->arrival = arrival;
  r->order = submitted_++;
  r->params = params;
  if (session) {
    r->session_id = *session;
    r->has_session = true;
  }
  r->chain = hasher_->chain(r->tokens.data(), r->tokens.size());
  return r;
}

std::vector<Event> EngineCore::abort(const std::string& rid, double now) {
  std::vector<Event> events;
  RequestPtr r = scheduler_.abort(rid);
  if (!r) return events;
  ++counters_["aborted_requests"];
  r->finished_at = now;
  finished_.push_back(record_of(*r));
  while (finished_.size() > max_request_records_) finished_.pop_front();
  Event e;
  e.rid = rid;
  e.kind = "done";
  e.finish_reason = "abort";
  e.t = now;
  events.push_back(e);
  return events;
}

Plan EngineCore::schedule(double now, std::vector<Event>& events) {
  Plan plan = scheduler_.schedule(now);
  for (const RequestPtr& r : plan.preempted) {
    Event e;
    e.rid = r->rid;
    e.kind = "preempted";
    e.t = now;
    events.push_back(e);
  }
  return plan;
}

void EngineCore::finish(const RequestPtr& r, const char* reason, double now,
                        std::vector<Event>& events) {
  r->state = RequestState::FINISHED;
  r->finish_reason = reason;
  r->finished_at = now;
  scheduler_.drop(r);
  ++counters_["finished_requests"];
  finished_.push_back(record_of(*r));
  while (finished_.size() > max_request_records_) finished_.pop_front();
  Event e;
  e.rid = r->rid;
  e.kind = "done";
  e.finish_reason = reason;
  e.t = now;
  events.push_back(e);
}

std::vector<Event> EngineCore::advance(const Plan& plan, const std::vector<int>& tokens,
                                       double now) {
  if (tokens.size() != plan.work.size()) {
    throw std::invalid_argument("advance: one token (or -1) per work item is required");
  }
  std::vector<Event> events;
  const int page = manager_->page_size();
  for (size_t i = 0; i < plan.work.size(); ++i) {
    const Work& w = plan.work[i];
    Request& r = *w.request;
    // The step wrote keys and values for the work's tokens: note it, offer the pages that
    // became full to the prefix index, give back what a window passed.
    r.num_computed = w.start + w.count;
    const int full = r.num_computed / page;
    if (manager_->prefix_sharing() && full > (int)r.chain.size()) {
      hasher_->extend(r.chain, r.tokens.data(), (size_t)r.num_computed);
    }
    manager_->commit(r.rid, r.chain, full);
    manager_->trim(r.rid, r.num_computed);
    if (!w.emits) continue;
    const int token = tokens[i];
    if (token < 0) throw std::invalid_argument("advance: '" + r.rid + "' completed its tokens but got none");
    Event e;
    e.rid = r.rid;
    e.kind = "token";
    e.token = token;
    e.index = r.num_out();
    e.t = now;
    r.append(token);
    if (std::isnan(r.first_token_at)) r.first_token_at = now;
    events.push_back(e);
    if (r.num_out() >= r.max_tokens) {
      finish(w.request, "length", now, events);
    } else if (!r.params.ignore_eos && eos_ids_.count(token)) {
      finish(w.request, "stop", now, events);
    }
  }
  return events;
}

void EngineCore::log_step(const Plan& plan, double now, double prepare_s, double forward_s,
                          double device_s, double step_s) {
  StepRecord rec;
  rec.t = now;
  rec.num_decode = plan.num_decode();
  rec.num_prefill = plan.num_prefill();
  rec.prefill_tokens = plan.num_prefill_tokens();
  rec.sched_s = plan.sched_seconds;
  rec.prepare_s = prepare_s;
  rec.forward_s = forward_s;
  rec.device_s = device_s;
  rec.step_s = step_s;
  rec.waiting = (int)scheduler_.waiting().size();
  rec.running = (int)scheduler_.running().size();
  rec.free_blocks = manager_->available();
  rec.preempted = (int)plan.preempted.size();
  steps_.push_back(rec);
  while (steps_.size() > max_step_records_) steps_.pop_front();
  ++counters_["steps"];
  counters_["prefill_requests"] += rec.num_prefill;
  counters_["prefill_tokens"] += rec.prefill_tokens;
  counters_["decode_tokens"] += rec.num_decode;
  counters_["preemptions"] += rec.preempted;
}

namespace {
double percentile(std::vector<double> values, double q) {
  if (values.empty()) return 0.0;
  std::sort(values.begin(), values.end());
  const double pos = (double)(values.size() - 1) * q;
  const size_t low = (size_t)pos;
  const size_t high = std::min(low + 1, values.size() - 1);
  return values[low] + (values[high] - values[low]) * (pos - (double)low);
}
}  // namespace

std::vector<std::pair<std::string, double>> EngineCore::summary() const {
  std::vector<std::pair<std::string, double>> out;
  for (const auto& kv : counters_) out.emplace_back(kv.first, (double)kv.second);
  std::vector<double> step_s, shares, decode_only;
  double sched = 0, prepare = 0, forward = 0, device = 0, total = 0;
  int max_running = 0, max_waiting = 0;
  for (const StepRecord& r : steps_) {
    step_s.push_back(r.step_s);
    total += r.step_s;
    sched += r.sched_s;
    prepare += r.prepare_s;
    forward += r.forward_s;
    device += r.device_s;
    if (r.step_s > 0) shares.push_back(r.sched_s / r.step_s);
    if (r.num_prefill == 0) decode_only.push_back(r.step_s);
    max_running = std::max(max_running, r.running);
    max_waiting = std::max(max_waiting, r.waiting);
  }
  const double n = (double)std::max<size_t>(1, steps_.size());
  const double whole = total > 0 ? total : 1e-9;
  out.emplace_back("wall_seconds", total);
  out.emplace_back("mean_step_ms", 1e3 * whole / n);
  out.emplace_back("p50_step_ms", 1e3 * percentile(step_s, 0.50));
  out.emplace_back("p99_step_ms", 1e3 * percentile(step_s, 0.99));
  out.emplace_back("mean_decode_step_ms",
                   decode_only.empty() ? 0.0
                                       : 1e3 * std::accumulate(decode_only.begin(), decode_only.end(), 0.0) /
                                             (double)decode_only.size());
  out.emplace_back("sched_seconds", sched);
  out.emplace_back("prepare_seconds", prepare);
  out.emplace_back("forward_seconds", forward);
  out.emplace_back("device_seconds", device);
  out.emplace_back("sched_share", sched / whole);
  out.emplace_back("prepare_share", prepare / whole);
  out.emplace_back("forward_share", forward / whole);
  out.emplace_back("p95_sched_share", percentile(shares, 0.95));
  out.emplace_back("mean_sched_us", 1e6 * sched / n);
  out.emplace_back("max_running_seen", (double)max_running);
  out.emplace_back("max_waiting_seen", (double)max_waiting);
  return out;
}

std::vector<RequestRecord> EngineCore::drain_finished() {
  std::vector<RequestRecord> out(finished_.begin(), finished_.end());
  finished_.clear();
  return out;
}

}  // namespace mercury
