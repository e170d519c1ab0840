"""An engine wired to the model-free executor and a clock the test drives
(same idea as reference tests/conftest.py:30-95)."""

from __future__ import annotations

from mercury_amd.cache import CacheManager
from mercury_amd.config import EngineConfig
from mercury_amd.engine.engine import Engine
from mercury_amd.parts import CacheSpec
from mercury_amd.testing import DeterministicExecutor, FakeClock

FULL = CacheSpec(kv_heads=2, head_dim=16, window=None)


class Harness:
    def __init__(self, engine, clock, executor):
        self.engine, self.clock, self.executor = engine, clock, executor
        self.events: dict = {}

    def submit(self, rid, prompt, max_tokens=4, **kwargs):
        bucket = self.events.setdefault(rid, [])
        self.engine.submit(rid, prompt, max_tokens, bucket.append, **kwargs)
        return rid

    def run(self, steps, dt=0.01):
        done = 0
        for _ in range(steps):
            if self.engine.step() is not None:
                done += 1
            self.clock.advance(dt)
        return done

    def drain(self, limit=100_000, dt=0.01):
        steps = 0
        while steps < limit:
            self.engine._drain_commands()
            if not self.engine.sched.has_work():
                break
            self.engine.step()
            self.clock.advance(dt)
            steps += 1
        return steps

    def tokens(self, rid):
        return [e.token for e in self.events.get(rid, []) if e.kind == "token"]

    def finish_reason(self, rid):
        for e in self.events.get(rid, []):
            if e.kind == "done":
                return e.finish_reason
        return None


def build(policy="fcfs", num_blocks=64, cache_slots=None, has_state=False, **overrides) -> Harness:
    cfg = EngineConfig(
        model="fake", num_blocks=num_blocks, block_size=overrides.pop("block_size", 16),
        max_running=overrides.pop("max_running", 8),
        prefill_budget=overrides.pop("prefill_budget", 8192),
        max_model_len=overrides.pop("max_model_len", 1024), policy=policy, **overrides)
    manager = CacheManager(cache_slots or {0: FULL}, cfg.num_blocks, cfg.block_size,
                           cfg.max_running, has_state)
    clock = FakeClock()
    executor = DeterministicExecutor(manager)
    return Harness(Engine(cfg, executor=executor, manager=manager, clock=clock), clock, executor)
