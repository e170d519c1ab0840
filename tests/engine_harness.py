"""The engine loop under test without a model: the model-free executor behind a real engine,
time that moves only when the test says so, and a journal of every event the engine sent."""

from __future__ import annotations

from mercury_amd.cache import CacheManager
from mercury_amd.config import EngineConfig
from mercury_amd.engine.engine import Engine
from mercury_amd.parts import CacheSpec
from mercury_amd.testing import DeterministicExecutor, ManualClock

FULL = CacheSpec(kv_heads=2, head_dim=16, window=None)
DEFAULTS = dict(block_size=16, max_running=8, prefill_budget=8192, max_model_len=1024)


class LoopUnderTest:
    """`journal` holds (request id, event) in the order the engine delivered them; the
    queries below read it."""

    def __init__(self, cfg: EngineConfig, cache_slots: dict, has_state: bool):
        self.clock = ManualClock()
        self.manager = CacheManager(cache_slots, cfg.num_blocks, cfg.block_size, cfg.max_running,
                                    has_state)
        self.executor = DeterministicExecutor(self.manager)
        self.engine = Engine(cfg, executor=self.executor, manager=self.manager, clock=self.clock)
        self.journal: list = []

    # ---- driving

    def submit(self, rid, prompt, max_tokens=4, **kwargs):
        self.engine.submit(rid, prompt, max_tokens,
                           lambda event, rid=rid: self.journal.append((rid, event)), **kwargs)
        return rid

    def run(self, passes: int, dt: float = 0.01) -> int:
        """`passes` passes of the loop, the clock moving `dt` after each; how many ran a step."""
        ran = 0
        for _ in range(passes):
            ran += self.engine.step() is not None
            self.clock.tick(dt)
        return ran

    def drain(self, dt: float = 0.01, limit: int = 100_000) -> int:
        """Passes until the engine has nothing queued or running (at most `limit`)."""
        ran = 0
        self.engine._take_commands()
        while self.engine.sched.has_work():
            assert ran < limit, "the loop did not come to rest"
            self.engine.step()
            self.clock.tick(dt)
            ran += 1
        return ran

    # ---- reading the journal

    def events_of(self, rid) -> list:
        return [event for who, event in self.journal if who == rid]

    @property
    def events(self) -> dict:
        out: dict = {}
        for who, event in self.journal:
            out.setdefault(who, []).append(event)
        return out

    def tokens(self, rid) -> list:
        return [e.token for e in self.events_of(rid) if e.kind == "token"]

    def finish_reason(self, rid):
        closing = [e.finish_reason for e in self.events_of(rid) if e.kind == "done"]
        return closing[-1] if closing else None


def build(policy="fcfs", num_blocks=64, cache_slots=None, has_state=False, **options) -> LoopUnderTest:
    settings = {**DEFAULTS, **options}
    cfg = EngineConfig(model="fake", num_blocks=num_blocks, policy=policy, **settings)
    return LoopUnderTest(cfg, cache_slots or {0: FULL}, has_state)
