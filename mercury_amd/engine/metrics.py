"""Per-step timings and a drainable log of finished requests
(reference: mercury/metrics.py:7-112)."""

from __future__ import annotations

from collections import deque
from dataclasses import astuple, dataclass, fields


@dataclass(slots=True)
class StepRecord:
    t: float
    num_prefill: int
    num_decode: int
    prefill_tokens: int
    sched_s: float
    prepare_s: float
    forward_s: float
    step_s: float
    waiting: int
    running: int
    free_blocks: int
    preempted: int


def percentile(values: list, q: float) -> float:
    if not values:
        return 0.0
    ordered = sorted(values)
    pos = (len(ordered) - 1) * q
    low = int(pos)
    high = min(low + 1, len(ordered) - 1)
    return ordered[low] + (ordered[high] - ordered[low]) * (pos - low)


class EngineMetrics:
    COUNTERS = ("steps", "idle_steps", "prefill_requests", "prefill_tokens", "decode_tokens",
                "finished_requests", "aborted_requests", "rejected_requests", "preemptions")

    def __init__(self, max_steps: int = 500_000, max_requests: int = 200_000):
        self.steps: deque = deque(maxlen=max_steps)
        self.finished: deque = deque(maxlen=max_requests)
        self.counters = {name: 0 for name in self.COUNTERS}
        self.started_at = None

    def add_step(self, record: StepRecord) -> None:
        self.steps.append(record)
        c = self.counters
        c["steps"] += 1
        c["prefill_requests"] += record.num_prefill
        c["prefill_tokens"] += record.prefill_tokens
        c["decode_tokens"] += record.num_decode
        c["preemptions"] += record.preempted

    def add_finished(self, record: dict) -> None:
        self.finished.append(record)

    def drain_finished(self) -> list:
        out = list(self.finished)
        self.finished.clear()
        return out

    def summary(self) -> dict:
        names = [f.name for f in fields(StepRecord)]
        cols = {n: [] for n in names}
        for record in self.steps:
            for name, value in zip(names, astuple(record)):
                cols[name].append(value)
        step_s, sched_s = cols["step_s"], cols["sched_s"]
        total = sum(step_s) or 1e-9
        decode_only = [t for t, p in zip(step_s, cols["num_prefill"]) if p == 0]
        shares = [s / t for s, t in zip(sched_s, step_s) if t > 0]
        return {
            **self.counters,
            "wall_seconds": sum(step_s),
            "mean_step_ms": 1e3 * total / max(1, len(step_s)),
            "p50_step_ms": 1e3 * percentile(step_s, 0.50),
            "p99_step_ms": 1e3 * percentile(step_s, 0.99),
            "mean_decode_step_ms": 1e3 * sum(decode_only) / len(decode_only) if decode_only else 0.0,
            "sched_seconds": sum(sched_s),
            "prepare_seconds": sum(cols["prepare_s"]),
            "forward_seconds": sum(cols["forward_s"]),
            "sched_share": sum(sched_s) / total,
            "prepare_share": sum(cols["prepare_s"]) / total,
            "forward_share": sum(cols["forward_s"]) / total,
            "p95_sched_share": percentile(shares, 0.95),
            "mean_sched_us": 1e6 * sum(sched_s) / max(1, len(sched_s)),
            "max_running_seen": max(cols["running"], default=0),
            "max_waiting_seen": max(cols["waiting"], default=0),
        }
