"""The engine loop over the model-free executor: events, finishing, aborts, limits, reuse of
freed room (vectors of reference tests/test_engine.py:12-181)."""

from __future__ import annotations

import random

import pytest

from mercury_amd.engine import SamplingParams
from mercury_amd.parts import CacheSpec
from tests.engine_harness import FULL, build


def test_every_request_emits_exactly_max_tokens_then_done_in_order():
    h = build(num_blocks=64, max_running=4)
    for i in range(12):
        h.submit(f"r{i}", list(range(i * 50, i * 50 + 40)), max_tokens=6)
    h.drain()
    for i in range(12):
        rid = f"r{i}"
        assert h.tokens(rid) == [h.executor.token_for(rid, k) for k in range(6)]
        assert h.finish_reason(rid) == "length"
        assert [e.index for e in h.events[rid] if e.kind == "token"] == list(range(6))


def test_hit_rate_matches_the_hand_computed_value():
    """Four requests share 64 tokens and add 16 private ones: 192 of 320 cached."""
    h = build(num_blocks=64)
    for i in range(4):
        h.submit(f"r{i}", list(range(64)) + [1000 + i] * 16, max_tokens=1)
        h.drain()
    stats = h.engine.manager.snapshot()
    assert (stats["query_tokens"], stats["hit_tokens"]) == (320, 192)
    assert stats["hit_rate"] == pytest.approx(0.6)


def test_a_partial_page_is_never_shared_and_output_extends_the_cache():
    h = build(num_blocks=64)
    for rid in "ab":
        h.submit(rid, list(range(24)), max_tokens=1)
        h.drain()
    assert h.engine.manager.snapshot()["hit_tokens"] == 16
    h.submit("c", list(range(500, 564)), max_tokens=40)
    h.drain()
    assert h.engine.manager.main_pool.num_cached_pages() > 1 + 4


def test_pages_become_shareable_only_once_their_tokens_are_computed():
    """With a 20-token budget a 64-token prompt is computed in four steps; a page enters the
    prefix cache when the step that filled it has run, not at admission."""
    h = build(num_blocks=64, prefill_budget=20)
    h.submit("a", list(range(64)), max_tokens=2)
    cached = []
    for _ in range(4):
        h.engine.step()
        cached.append(h.engine.manager.main_pool.num_cached_pages())
    assert cached == [1, 2, 3, 4]


def test_aborts_return_pages_and_silence_the_request():
    h = build(num_blocks=32, max_running=2)
    for i in range(6):
        h.submit(f"r{i}", list(range(i * 100, i * 100 + 48)), max_tokens=50)
    h.run(3)
    h.engine.abort("r0")
    h.engine.abort("r5")                                 # still waiting: never runs
    h.drain()
    assert h.engine.metrics.counters["aborted_requests"] == 2
    assert h.finish_reason("r0") == "abort" and h.finish_reason("r5") == "abort"
    assert h.tokens("r5") == [] and h.engine.leaked_blocks() == 0


def test_a_tenth_of_requests_cancelled_leaks_nothing():
    rng = random.Random(3)
    h = build(num_blocks=64, max_running=6, prefill_budget=96)
    cancelled = 0
    for i in range(300):
        h.submit(f"r{i}", [rng.randrange(40)] * 16 + [rng.randrange(9000) for _ in range(rng.randrange(1, 60))],
                 max_tokens=rng.randrange(4, 24))
        h.engine.step()
        h.clock.tick(0.01)
        if rng.random() < 0.1:
            live = [r.rid for r in h.engine.sched.running + h.engine.sched.waiting]
            if live:
                h.engine.abort(rng.choice(live))
                cancelled += 1
    h.drain()
    assert cancelled > 15 and h.engine.metrics.counters["aborted_requests"] >= cancelled - 2
    assert h.engine.leaked_blocks() == 0
    h.engine.manager.check_invariants()


def test_requests_that_cannot_fit_are_rejected_not_queued():
    h = build(num_blocks=4, max_model_len=1024)
    h.submit("huge", list(range(200)), max_tokens=10)
    h.submit("empty", [], max_tokens=4)
    h.drain()
    assert [e.kind for e in h.events["huge"]] == ["error"] and "ceiling" in h.events["huge"][0].message
    assert [e.kind for e in h.events["empty"]] == ["error"]
    assert h.engine.sched.waiting == [] and h.engine.metrics.counters["rejected_requests"] == 2


def test_a_freed_place_is_taken_on_the_very_next_step():
    h = build(num_blocks=64, max_running=2)
    h.submit("a", list(range(32)), max_tokens=2)
    h.submit("b", list(range(100, 132)), max_tokens=20)
    h.submit("c", list(range(200, 232)), max_tokens=4)
    h.engine.step()
    assert len(h.engine.sched.running) == 2 and h.engine.sched.waiting[0].rid == "c"
    h.engine.step()
    assert h.finish_reason("a") == "length"
    h.engine.step()
    assert any(r.rid == "c" for r in h.engine.sched.running)


def test_stop_on_eos_unless_ignored():
    h = build(num_blocks=64)
    rid = "stopper"
    eos = h.executor.token_for(rid, 2)
    h.engine.eos_ids = {eos}
    h.submit(rid, list(range(20)), max_tokens=10)
    h.submit("deaf", list(range(20)), max_tokens=5, params=SamplingParams(ignore_eos=True))
    h.engine.eos_ids |= {h.executor.token_for("deaf", 1)}
    h.drain()
    assert len(h.tokens(rid)) == 3 and h.finish_reason(rid) == "stop"
    assert len(h.tokens("deaf")) == 5 and h.finish_reason("deaf") == "length"


def test_a_sink_that_raises_aborts_its_request():
    h = build(num_blocks=64)

    def broken(event):
        raise ConnectionError("client went away")

    h.engine.submit("gone", list(range(30)), 50, broken)
    h.submit("fine", list(range(30)), max_tokens=5)
    h.drain()
    assert len(h.tokens("fine")) == 5 and h.engine.leaked_blocks() == 0
    assert h.engine.metrics.counters["aborted_requests"] == 1


def test_preempted_requests_hear_about_it_and_still_finish():
    h = build(num_blocks=11, max_running=4, max_model_len=176)
    for i in range(4):
        h.submit(f"r{i}", list(range(i * 100, i * 100 + 80)), max_tokens=24)
    h.drain()
    kinds = [e.kind for rid in h.events for e in h.events[rid]]
    assert "preempted" in kinds
    assert all(len(h.tokens(f"r{i}")) == 24 for i in range(4)) and h.engine.leaked_blocks() == 0


def test_state_slots_and_window_groups_through_the_loop():
    slots = {0: FULL, 1: CacheSpec(2, 16, window=40)}
    h = build(num_blocks=40, max_running=3, prefill_budget=50, cache_slots=slots, has_state=True,
              debug_invariants=True)
    for i in range(9):
        h.submit(f"r{i}", list(range(i, i + 70 + 9 * i)), max_tokens=30)
    h.drain()
    assert h.engine.metrics.counters["finished_requests"] == 9
    assert h.engine.leaked_blocks() == 0
    assert h.engine.manager.state_slots.num_available() == 3
    assert h.engine.manager.snapshot()["hit_tokens"] == 0     # no prefix sharing with state


def test_generate_blocks_until_every_prompt_is_done():
    h = build(num_blocks=64, max_running=2)
    out = h.engine.generate([list(range(10)), list(range(40)), [5]], max_tokens=[3, 1, 4])
    assert [len(o) for o in out] == [3, 1, 4]
    with pytest.raises(ValueError, match="ceiling"):
        h.engine.generate([list(range(2000))], max_tokens=5)


def test_snapshot_and_step_log():
    h = build(policy="lpm_aging", num_blocks=32, max_running=1)
    h.submit("a", list(range(32)), max_tokens=3)
    h.clock.tick(0.5)
    h.submit("b", list(range(100, 132)), max_tokens=3)
    h.drain()
    snap = h.engine.snapshot()
    assert snap["config"]["policy"] == "lpm_aging" and snap["config"]["kv_capacity_tokens"] == 512
    assert snap["allocator"]["num_blocks"] == 32 and snap["engine"]["decode_tokens"] > 0
    assert 0.0 <= snap["engine"]["sched_share"] <= 1.0
    records = {r["rid"]: r for r in h.engine.drain_request_records()}
    assert records["b"]["queue_delay"] > 0.0 and records["b"]["output_tokens"] == 3
