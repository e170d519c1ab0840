"""What the engine calls once per step: run the plan's tokens, sample, return tokens.

The engine depends on `execute(plan) -> ExecResult` only, so that the scheduler, the cache
manager and the engine loop can be exercised against a model-free stand-in
(reference: mercury/runner.py:40-41, mercury/testing.py).
"""

from __future__ import annotations

import time
from dataclasses import dataclass, field

from .batch import SeqChunk


@dataclass
class ExecResult:
    """tokens[i] is the sampled token of plan.work[i], or None when that work item did not
    complete its sequence (a prompt portion that is not the last)."""

    tokens: list = field(default_factory=list)
    prepare_seconds: float = 0.0      # packing the step and copying it to the device (host)
    forward_seconds: float = 0.0      # the rest of the host's wall clock, the wait included
    device_seconds: float = 0.0       # the step's kernels, by events on the device


class _Pending:
    """Tokens on their way from the device into pinned host memory: `wait()` gives them as a
    list.  `began` is the event recorded before the step's first kernel, `previous` the event
    that closed the step before this one on the same stream."""

    def __init__(self, tokens_dev, host, done, began=None, previous=None):
        self.host, self.done, self.began = host[:tokens_dev.shape[0]], done, began
        self.previous = previous
        self.host.copy_(tokens_dev, non_blocking=True)
        self.done.record()

    def wait(self) -> list:
        self.done.synchronize()
        return self.host.tolist()

    def device_seconds(self) -> float:
        """Time on the device from the step's start to its tokens' copy (after wait).  A step
        launched ahead has its start event recorded while the step before it still runs; the
        stream reaches that event only when the earlier step is done, but the step's own time
        cannot begin before the earlier step's end either way: the later of the two counts, so
        that the steps' times never overlap and add up to no more than the wall clock."""
        if self.began is None:
            return 0.0
        own = self.began.elapsed_time(self.done)
        if self.previous is not None:
            own = min(own, self.previous.elapsed_time(self.done))
        return 1e-3 * max(own, 0.0)


class _PinnedRing:
    """A few pinned int32 buffers and events, used in turn: allocating pinned memory for every
    step costs far more than a step's host work.  A buffer comes round again after `depth`
    uses; at most two results are ever in flight."""

    def __init__(self, size: int, depth: int = 4):
        import torch

        self.size = size
        self.buffers = [torch.empty(size, dtype=torch.int32, pin_memory=True) for _ in range(depth)]
        self.events = [torch.cuda.Event(enable_timing=True) for _ in range(depth)]
        self.starts = [torch.cuda.Event(enable_timing=True) for _ in range(depth)]
        self.next = 0
        self.last_done = None      # the event that closed the most recent step

    def begin(self):
        """Record, now, the start event of the step whose tokens the next `pending` carries."""
        self.starts[self.next].record()

    def pending(self, tokens_dev) -> _Pending:
        import torch

        n = tokens_dev.shape[0]
        i = self.next
        self.next = (i + 1) % len(self.buffers)
        previous = self.last_done
        if n > self.size:
            made = _Pending(tokens_dev, torch.empty(n, dtype=torch.int32, pin_memory=True),
                            torch.cuda.Event(enable_timing=True), self.starts[i], previous)
        else:
            made = _Pending(tokens_dev, self.buffers[i], self.events[i], self.starts[i], previous)
        self.last_done = made.done
        return made


@dataclass
class _Ahead:
    """A decode step started before the plan that asks for it exists."""

    rids: tuple
    starts: tuple
    fed: list | None         # the token ids it ran on, once the host knows them
    tokens_dev: object
    pending: _Pending


class GpuExecutor:
    """The real thing: the step function over the plan's work, then the sampler.

    With `lookahead`, a plan the scheduler calls steady (the same requests decoding on) has
    its successor started at once: the sampled tokens stay on the device as the next step's
    input, the pages the next positions need are taken now, and the graph of the next step is
    launched before this step's tokens are read.  The next `execute` finds its work in
    flight if its plan is the expected one (same requests in the same order, each one token
    further, fed the tokens that were sampled); otherwise what ran ahead is dropped: it wrote
    keys and values only at positions past what any request has computed, which the step
    that really computes them writes again."""

    def __init__(self, runner, sampler, lookahead: bool = False):
        self.runner, self.sampler = runner, sampler
        self.model_config = runner.model.config
        self.kv_bytes = runner.kv_bytes
        manager = runner.manager
        self.lookahead = (bool(lookahead) and runner.use_graphs
                          and not runner.states and all(g.window is None for g in manager.groups))
        self._ahead: _Ahead | None = None
        self._ring = _PinnedRing(max(256, runner.max_graph_batch))
        self.stats = {"ahead_started": 0, "ahead_used": 0}

    def execute(self, plan) -> ExecResult:
        started = time.perf_counter()
        ahead, self._ahead = self._ahead, None
        work = plan.work
        if ahead is not None and self._matches(ahead, work):
            tokens_dev, pending = ahead.tokens_dev, ahead.pending
            self.stats["ahead_used"] += 1
            self.runner.last_prepare_seconds = 0.0
        else:
            self._ring.begin()
            logits = self.runner.step_plan(plan)
            emitting = plan.emitting
            tokens_dev = self.sampler.launch(logits, emitting) if emitting else None
            pending = self._ring.pending(tokens_dev) if emitting else None
        if self.lookahead and plan.steady:
            self._ahead = self._start_ahead(work, tokens_dev)
        if pending is None:
            import torch

            torch.cuda.current_stream(self.runner.device).synchronize()
        sampled = iter(pending.wait() if pending is not None else ())
        result = ExecResult(tokens=[next(sampled) if w.emits else None for w in work])
        if self._ahead is not None:
            self._ahead.fed = result.tokens
        result.prepare_seconds = self.runner.last_prepare_seconds
        result.forward_seconds = time.perf_counter() - started - result.prepare_seconds
        if pending is not None:
            result.device_seconds = pending.device_seconds()
        return result

    @staticmethod
    def _matches(ahead: _Ahead, work: list) -> bool:
        if len(work) != len(ahead.rids) or ahead.fed is None:
            return False
        for w, rid, start, token in zip(work, ahead.rids, ahead.starts, ahead.fed):
            r = w.request
            if (r.rid != rid or w.start != start or w.count != 1 or not w.emits
                    or r.token_at(start) != token):
                return False
        return True

    def _start_ahead(self, work: list, tokens_dev) -> _Ahead | None:
        """Launch the step after this one for the same requests, fed this step's tokens from
        the device.  None when there is no captured graph for it yet (capturing is left to the
        step that is asked for) or a page the next positions need cannot be had."""
        manager = self.runner.manager
        chunks = [SeqChunk(w.request.rid, [0], w.start + 1, [0]) for w in work]
        if not self.runner.captured(len(chunks), max(c.start for c in chunks) + 1):
            return None
        if any(c.start + 1 > self.runner.max_model_len for c in chunks):
            return None
        new_pages = sum(1 for c in chunks if c.start % manager.page_size == 0)
        if new_pages > manager.num_available():
            return None
        for c in chunks:
            if not manager.grow(c.key, c.start, c.start + 1):
                return None
        self._ring.begin()
        logits = self.runner.step_ahead(chunks, tokens_dev)
        requests = [w.request for w in work]
        next_dev = self.sampler.launch(logits, requests, ahead=1)
        self.stats["ahead_started"] += 1
        return _Ahead(tuple(r.rid for r in requests), tuple(c.start for c in chunks), None,
                      next_dev, self._ring.pending(next_dev))

    def snapshot(self) -> dict:
        r = self.runner
        return {"device": str(r.device), "dtype": str(r.dtype).replace("torch.", ""),
                "kv_bytes": r.kv_bytes, "cache_slots": len(r.kv),
                "kv_bytes_per_token": r.kv_bytes_per_token(), "memory": r.memory_report(),
                "lookahead": dict(self.stats)}
