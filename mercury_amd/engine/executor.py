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
    prepare_seconds: float = 0.0
    forward_seconds: float = 0.0


class GpuExecutor:
    """The real thing: the step function over the plan's work, then the sampler."""

    def __init__(self, runner, sampler):
        self.runner, self.sampler = runner, sampler
        self.model_config = runner.model.config
        self.kv_bytes = runner.kv_bytes

    def execute(self, plan) -> ExecResult:
        import torch

        started = time.perf_counter()
        chunks = []
        for w in plan.work:
            tokens = w.request.tokens[w.start:w.start + w.count]
            chunks.append(SeqChunk(w.request.rid, tokens, w.start, [w.count - 1] if w.emits else []))
        logits = self.runner.step(chunks)
        emitting = [w.request for w in plan.work if w.emits]
        sampled = iter(self.sampler.sample(logits, emitting))
        result = ExecResult(tokens=[next(sampled) if w.emits else None for w in plan.work])
        torch.cuda.synchronize()
        result.prepare_seconds = self.runner.last_prepare_seconds
        result.forward_seconds = time.perf_counter() - started - result.prepare_seconds
        return result

    def snapshot(self) -> dict:
        r = self.runner
        return {"device": str(r.device), "dtype": str(r.dtype).replace("torch.", ""),
                "kv_bytes": r.kv_bytes, "cache_slots": len(r.kv),
                "kv_bytes_per_token": r.kv_bytes_per_token()}
