"""The scheduler: one pass per engine step that decides which tokens run.

Every step it (1) gives each running request its next tokens, one token when it is decoding,
a portion of its prompt under the step's token budget when it is still prefilling, taking
pages as needed and preempting the newest admitted request when a pool is empty; (2) admits
waiting requests in policy order while there is room, budget and memory
(reference: mercury/scheduler.py:122-179, which admits whole prompts only; the three policies
and what each does when the head of the queue does not fit are the reference's,
mercury/scheduler.py:103-120, :155-160).

When pages run out: the newest admitted request loses everything it holds and goes back to
the waiting queue at its original arrival time; it later starts over with prompt + generated
tokens as its prompt (reference: mercury/scheduler.py:91-101).
"""

from __future__ import annotations

import bisect
import time
from dataclasses import dataclass, field

from .request import Request, RequestState


@dataclass
class Work:
    """Tokens [start, start + count) of a request run this step; `emits` when they complete
    the sequence, so the step's last logits give the request's next token."""

    request: Request
    start: int
    count: int
    emits: bool


@dataclass
class Plan:
    work: list = field(default_factory=list)
    preempted: list = field(default_factory=list)
    admitted: list = field(default_factory=list)
    sched_seconds: float = 0.0
    # The next plan is expected to be this one a token further: every request decodes and
    # none reaches its length limit with this step's token, and nobody waits for a place that
    # is free.  (A stop token may still prove it wrong.)  An executor may use it to start the
    # next step's work early.
    steady: bool = False

    def __bool__(self) -> bool:
        return bool(self.work)

    @property
    def prefill(self) -> list:
        return [w.request for w in self.work if w.count > 1 or not w.emits or w.start < w.request.prompt_len]

    @property
    def decode(self) -> list:
        return [w.request for w in self.work if w.count == 1 and w.emits and w.start >= w.request.prompt_len]

    @property
    def num_prefill_tokens(self) -> int:
        decode = {id(r) for r in self.decode}
        return sum(w.count for w in self.work if id(w.request) not in decode)


class Scheduler:
    def __init__(self, manager, hasher, policy: str = "fcfs", max_running: int = 64,
                 prefill_budget: int = 8192, aging_tokens_per_s: float = 2000.0,
                 max_wait_s: float = 5.0, scan_limit: int = 128):
        self.manager, self.hasher = manager, hasher
        self.policy = policy
        self.max_running = max_running
        self.prefill_budget = prefill_budget
        self.aging = aging_tokens_per_s
        self.max_wait_s = max_wait_s
        self.scan_limit = scan_limit
        self.waiting: list = []
        self.running: list = []
        self.stats = {"steps": 0, "sched_seconds": 0.0, "preemptions": 0, "admissions": 0,
                      "max_waiting": 0, "scan_limit_exceeded": 0, "scored_requests": 0}

    # ---- queue operations

    def add(self, r: Request) -> None:
        r.state = RequestState.WAITING
        bisect.insort(self.waiting, r, key=lambda x: x.arrival)

    def _release(self, r: Request) -> None:
        if self.manager.holds(r.rid):
            self.manager.free(r.rid)

    def abort(self, rid: str):
        for queue in (self.waiting, self.running):
            for r in queue:
                if r.rid == rid:
                    queue.remove(r)
                    self._release(r)
                    r.state = RequestState.ABORTED
                    r.finish_reason = "abort"
                    return r
        return None

    def drop(self, r: Request) -> None:
        """Finished: everything it holds goes back; committed pages stay findable."""
        if r in self.running:
            self.running.remove(r)
        elif r in self.waiting:
            self.waiting.remove(r)
        self._release(r)

    def has_work(self) -> bool:
        return bool(self.waiting or self.running)

    def _preempt(self, r: Request) -> None:
        self.running.remove(r)
        self._release(r)
        r.num_computed = 0
        r.num_cached = 0
        r.preemptions += 1
        r.hashes = self.hasher.hashes(r.tokens)
        self.stats["preemptions"] += 1
        self.add(r)

    # ---- policy

    def _score(self, r: Request, now: float) -> float:
        """Admission priority, high first (reference: mercury/scheduler.py:103-120)."""
        if self.policy == "fcfs":
            return -r.arrival
        cached = self.manager.cached_prefix_tokens(r.hashes)
        if self.policy == "lpm":
            return float(cached)
        waited = now - r.arrival
        if waited >= self.max_wait_s:
            return float("inf")
        return cached + self.aging * waited

    # ---- the pass

    def schedule(self, now: float) -> Plan:
        t0 = time.perf_counter()
        plan = Plan()
        budget = self.prefill_budget

        # 1. Running requests, oldest admission first.
        for r in list(self.running):
            if not r.running:
                continue  # preempted while an earlier request took pages
            remaining = r.remaining
            count = 1 if remaining == 1 else min(remaining, budget)
            if count <= 0:
                continue  # mid-prompt and the step's budget is spent
            while r.running and not self.manager.grow(r.rid, r.num_computed, r.num_computed + count):
                victim = self.running[-1]
                self._preempt(victim)
                plan.preempted.append(victim)
            if not r.running:
                continue
            if remaining > 1:
                budget -= count
            plan.work.append(Work(r, r.num_computed, count, count == remaining))
        if plan.preempted:
            gone = {id(v) for v in plan.preempted}
            plan.work = [w for w in plan.work if id(w.request) not in gone]

        # 2. Admission in policy order.
        head, tail = self.waiting[: self.scan_limit], self.waiting[self.scan_limit:]
        if tail:
            self.stats["scan_limit_exceeded"] += 1
        self.stats["scored_requests"] += len(head)
        order = sorted(head, key=lambda r: (-self._score(r, now), r.arrival)) + tail
        for r in order:
            if len(self.running) + len(plan.admitted) >= self.max_running or budget <= 0:
                break
            cached = self.manager.admit(r.rid, r.hashes, r.seq_len)
            if cached is None:
                starving = self.policy == "lpm_aging" and self._score(r, now) == float("inf")
                if self.policy == "fcfs" or starving:
                    break
                continue
            r.num_cached = r.num_computed = cached
            count = min(r.remaining, budget)
            if not self.manager.grow(r.rid, r.num_computed, r.num_computed + count):
                self.manager.free(r.rid)   # a windowed group had no page for the first portion
                r.num_cached = r.num_computed = 0
                if self.policy == "fcfs":
                    break
                continue
            r.state = RequestState.RUNNING
            r.last_admitted_at = now
            if r.admitted_at is None:
                r.admitted_at = now
            r.recomputed_tokens += r.seq_len - cached
            budget -= count
            plan.admitted.append(r)
            plan.work.append(Work(r, r.num_computed, count, count == r.remaining))

        if plan.admitted:
            taken = {id(r) for r in plan.admitted}
            self.waiting = [r for r in self.waiting if id(r) not in taken]
            self.running.extend(plan.admitted)
            self.stats["admissions"] += len(plan.admitted)

        plan.steady = (bool(plan.work) and not plan.preempted
                       and (not self.waiting or len(self.running) >= self.max_running)
                       and all(w.count == 1 and w.emits and w.start >= w.request.prompt_len
                               and len(w.request.out) + 1 < w.request.max_tokens
                               for w in plan.work))
        plan.sched_seconds = time.perf_counter() - t0
        self.stats["steps"] += 1
        self.stats["sched_seconds"] += plan.sched_seconds
        self.stats["max_waiting"] = max(self.stats["max_waiting"], len(self.waiting))
        return plan

    def snapshot(self) -> dict:
        steps = self.stats["steps"] or 1
        return {"policy": self.policy, "waiting": len(self.waiting), "running": len(self.running),
                "mean_sched_seconds": self.stats["sched_seconds"] / steps, **self.stats}
