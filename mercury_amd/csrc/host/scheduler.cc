#include "scheduler.h"

#include <algorithm>
#include <chrono>

namespace mercury {

const char* state_name(RequestState s) {
  switch (s) {
    case RequestState::WAITING: return "waiting";
    case RequestState::RUNNING: return "running";
    case RequestState::FINISHED: return "finished";
    default: return "aborted";
  }
}

Policy parse_policy(const std::string& name) {
  if (name == "fcfs") return Policy::FCFS;
  if (name == "lpm") return Policy::LPM;
  if (name == "lpm_aging") return Policy::LPM_AGING;
  throw std::invalid_argument("policy must be one of fcfs, lpm, lpm_aging, got '" + name + "'");
}

int Plan::num_decode() const {
  int n = 0;
  for (const Work& w : work) n += w.decode();
  return n;
}

int Plan::num_prefill_tokens() const {
  int n = 0;
  for (const Work& w : work) {
    if (!w.decode()) n += w.count;
  }
  return n;
}

Scheduler::Scheduler(std::shared_ptr<CacheManager> manager, std::shared_ptr<PageHasher> hasher,
                     SchedulerOptions options)
    : manager_(std::move(manager)), hasher_(std::move(hasher)), options_(options) {}

void Scheduler::add(const RequestPtr& r) {
  r->state = RequestState::WAITING;
  auto later = [](const RequestPtr& a, const RequestPtr& b) {
    return a->arrival < b->arrival || (a->arrival == b->arrival && a->order < b->order);
  };
  waiting_.insert(std::upper_bound(waiting_.begin(), waiting_.end(), r, later), r);
}

void Scheduler::release(const Request& r) {
  if (manager_->holds(r.rid)) manager_->release(r.rid);
}

RequestPtr Scheduler::abort(const std::string& rid) {
  for (std::vector<RequestPtr>* queue : {&waiting_, &running_}) {
    for (auto it = queue->begin(); it != queue->end(); ++it) {
      if ((*it)->rid != rid) continue;
      RequestPtr r = *it;
      queue->erase(it);
      release(*r);
      r->state = RequestState::ABORTED;
      r->finish_reason = "abort";
      return r;
    }
  }
  return nullptr;
}

void Scheduler::drop(const RequestPtr& r) {
  auto gone = [&](std::vector<RequestPtr>& queue) {
    auto it = std::find(queue.begin(), queue.end(), r);
    if (it == queue.end()) return false;
    queue.erase(it);
    return true;
  };
  if (!gone(running_)) gone(waiting_);
  release(*r);
}

void Scheduler::preempt(const RequestPtr& r) {
  running_.erase(std::find(running_.begin(), running_.end(), r));
  release(*r);
  r->num_computed = 0;
  r->num_cached = 0;
  ++r->preemptions;
  r->chain = hasher_->chain(r->tokens.data(), r->tokens.size());
  ++stats_.preemptions;
  add(r);
}

double Scheduler::score(const Request& r, double now) const {
  if (options_.policy == Policy::FCFS) return -r.arrival;
  const double cached = (double)manager_->cached_prefix_tokens(r.chain);
  if (options_.policy == Policy::LPM) return cached;
  const double waited = now - r.arrival;
  if (waited >= options_.max_wait_s) return std::numeric_limits<double>::infinity();
  return cached + options_.aging_tokens_per_s * waited;
}

// Running requests, oldest admission first: a decoding request gets its one token, a request
// still in its prompt as much of it as the step's budget has left.
void Scheduler::continue_running(Plan& plan, int& budget) {
  const std::vector<RequestPtr> order = running_;       // preemption edits running_
  for (const RequestPtr& r : order) {
    if (!r->running()) continue;                        // preempted for an earlier request
    const int remaining = r->remaining();
    const int count = remaining == 1 ? 1 : std::min(remaining, budget);
    if (count <= 0) continue;                           // mid-prompt and the budget is spent
    while (r->running() && !manager_->grow(r->rid, r->num_computed, r->num_computed + count)) {
      RequestPtr victim = running_.back();
      preempt(victim);
      plan.preempted.push_back(victim);
    }
    if (!r->running()) continue;
    if (remaining > 1) budget -= count;
    plan.work.push_back(Work{r, r->num_computed, count, count == remaining});
  }
  if (!plan.preempted.empty()) {
    auto lost = [&](const Work& w) {
      return std::find(plan.preempted.begin(), plan.preempted.end(), w.request) != plan.preempted.end();
    };
    plan.work.erase(std::remove_if(plan.work.begin(), plan.work.end(), lost), plan.work.end());
  }
}

void Scheduler::admit_waiting(Plan& plan, int& budget, double now) {
  const size_t scanned = std::min(waiting_.size(), (size_t)std::max(0, options_.scan_limit));
  if (scanned < waiting_.size()) ++stats_.scan_limit_exceeded;
  stats_.scored_requests += (int64_t)scanned;
  struct Ranked { double score; RequestPtr r; };
  std::vector<Ranked> ranked;
  ranked.reserve(waiting_.size());
  for (size_t i = 0; i < scanned; ++i) ranked.push_back({score(*waiting_[i], now), waiting_[i]});
  // high score first; the queue's own order (arrival) among equals
  std::stable_sort(ranked.begin(), ranked.end(),
                   [](const Ranked& a, const Ranked& b) { return a.score > b.score; });
  for (size_t i = scanned; i < waiting_.size(); ++i) ranked.push_back({0.0, waiting_[i]});

  const double inf = std::numeric_limits<double>::infinity();
  for (const Ranked& entry : ranked) {
    const RequestPtr& r = entry.r;
    if ((int)(running_.size() + plan.admitted.size()) >= options_.max_running || budget <= 0) break;
    const int cached = manager_->admit(r->rid, r->chain, r->seq_len());
    if (cached < 0) {
      const bool starving = options_.policy == Policy::LPM_AGING && score(*r, now) == inf;
      if (options_.policy == Policy::FCFS || starving) break;
      continue;
    }
    r->num_cached = r->num_computed = cached;
    const int count = std::min(r->remaining(), budget);
    if (!manager_->grow(r->rid, r->num_computed, r->num_computed + count)) {
      manager_->release(r->rid);     // a windowed group had no page for the first portion
      r->num_cached = r->num_computed = 0;
      if (options_.policy == Policy::FCFS) break;
      continue;
    }
    r->state = RequestState::RUNNING;
    r->last_admitted_at = now;
    if (std::isnan(r->admitted_at)) r->admitted_at = now;
    r->recomputed_tokens += r->seq_len() - cached;
    budget -= count;
    plan.admitted.push_back(r);
    plan.work.push_back(Work{r, r->num_computed, count, count == r->remaining()});
  }
  if (!plan.admitted.empty()) {
    auto taken = [&](const RequestPtr& r) {
      return std::find(plan.admitted.begin(), plan.admitted.end(), r) != plan.admitted.end();
    };
    waiting_.erase(std::remove_if(waiting_.begin(), waiting_.end(), taken), waiting_.end());
    running_.insert(running_.end(), plan.admitted.begin(), plan.admitted.end());
    stats_.admissions += (int64_t)plan.admitted.size();
  }
}

Plan Scheduler::schedule(double now) {
  const auto t0 = std::chrono::steady_clock::now();
  Plan plan;
  int budget = options_.prefill_budget;
  continue_running(plan, budget);
  admit_waiting(plan, budget, now);

  plan.steady = !plan.work.empty() && plan.preempted.empty() &&
                (waiting_.empty() || (int)running_.size() >= options_.max_running);
  for (const Work& w : plan.work) {
    if (!plan.steady) break;
    plan.steady = w.decode() && w.request->num_out() + 1 < w.request->max_tokens;
  }
  plan.sched_seconds =
      std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count();
  ++stats_.steps;
  stats_.sched_seconds += plan.sched_seconds;
  stats_.max_waiting = std::max<int64_t>(stats_.max_waiting, (int64_t)waiting_.size());
  return plan;
}

}  // namespace mercury
