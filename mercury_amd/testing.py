"""Model-free stand-ins for tests of the scheduler, the cache manager and the engine loop
(reference: mercury/testing.py:20-78)."""

from __future__ import annotations

import time
import zlib

from .engine.executor import ExecResult


def stand_in_token(rid: str, index: int, vocab_size: int) -> int:
    """The token the model-free executor emits as output `index` of request `rid`: a fixed
    function of the two, so a test can say what a request must have produced however its
    work was scheduled."""
    return (zlib.crc32(rid.encode()) + 7919 * index) % vocab_size


class DeterministicExecutor:
    """Produces `stand_in_token(rid, index, vocab)` without a model, after checking what
    the real step function relies on: every work item starts where the request's computed
    tokens end and the request holds pages for all positions it touches, no page twice."""

    def __init__(self, manager=None, vocab_size: int = 32000, step_delay: float = 0.0):
        self.manager = manager
        self.vocab_size = vocab_size
        self.step_delay = step_delay
        self.model_config = None
        self.kv_bytes = 0
        self.steps = self.prefill_tokens_seen = self.decode_tokens_seen = 0

    def token_for(self, rid: str, index: int) -> int:
        return stand_in_token(rid, index, self.vocab_size)

    def _check(self, work) -> None:
        r = work.request
        if work.start != r.num_computed:
            raise AssertionError(f"{r.rid}: work starts at {work.start}, computed {r.num_computed}")
        if work.count <= 0 or work.start + work.count > r.seq_len:
            raise AssertionError(f"{r.rid}: work [{work.start}, +{work.count}) outside the sequence")
        if work.emits != (work.start + work.count == r.seq_len):
            raise AssertionError(f"{r.rid}: emits flag does not match the end of the sequence")
        if self.manager is None:
            return
        ps = self.manager.page_size
        for gi, group in enumerate(self.manager.groups):
            table = self.manager.table(r.rid, gi)
            need = -(-(work.start + work.count) // ps)
            if len(table) < need:
                raise AssertionError(f"{r.rid}: {len(table)} pages cover less than {need}")
            first = 0 if group.window is None else \
                max(0, work.start - group.window + 1) // ps
            live = table[first:need]
            if any(p < 0 for p in live):
                raise AssertionError(f"{r.rid}: a page the step reads was given back")
            if len(set(live)) != len(live):
                raise AssertionError(f"{r.rid}: the same page appears twice in {live}")

    def execute(self, plan) -> ExecResult:
        started = time.perf_counter()
        tokens = []
        for w in plan.work:
            self._check(w)
            tokens.append(self.token_for(w.request.rid, w.request.num_out) if w.emits else None)
        self.steps += 1
        self.prefill_tokens_seen += plan.num_prefill_tokens
        self.decode_tokens_seen += plan.num_decode
        if self.step_delay:
            time.sleep(self.step_delay)
        return ExecResult(tokens=tokens, forward_seconds=time.perf_counter() - started)

    def snapshot(self) -> dict:
        return {"device": "none", "executor": "model-free", "steps": self.steps,
                "prefill_tokens": self.prefill_tokens_seen, "decode_tokens": self.decode_tokens_seen}


class ManualClock:
    """Time that stands still until the test moves it with `tick`; calling it reads it.  The
    scheduler's waiting times and deadlines then depend on the test alone."""

    def __init__(self, at: float = 0.0):
        self.at = float(at)

    def __call__(self) -> float:
        return self.at

    def tick(self, seconds: float) -> float:
        self.at += seconds
        return self.at
