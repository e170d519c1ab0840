"""The scheduler's decisions: policy order, what happens when the head of the queue does not
fit, prompts cut into portions under the token budget, preemption when pages run out
(vectors of reference tests/test_scheduler.py:34-190 plus the portions the reference lacks)."""

from __future__ import annotations

import random

from mercury_amd.cache import CacheManager, PageHasher
from mercury_amd.engine import Request, RequestState
from mercury_amd.engine import Scheduler
from mercury_amd.parts import CacheSpec
from tests.engine_harness import FULL, build

PS = 16
H = PageHasher(PS)


def make(num_pages, policy="fcfs", max_running=8, slots=None, **kw):
    manager = CacheManager(slots or {0: FULL}, num_pages, PS, 64)
    return manager, Scheduler(manager, H, policy=policy, max_running=max_running, **kw)


def request(rid, prompt, arrival, max_tokens=8):
    return Request(rid=rid, prompt=list(prompt), max_tokens=max_tokens, arrival=arrival,
                   hashes=H.hashes(prompt))


def warm(manager, tokens):
    hashes = H.hashes(tokens)
    manager.admit("warm", hashes, len(tokens))
    manager.commit("warm", hashes, len(tokens) // PS)
    manager.free("warm")


def finish_step(plan):
    """What the engine does after executing a plan, without a model."""
    for w in plan.work:
        w.request.num_computed = w.start + w.count
        if w.emits:
            w.request.append(1)


def rids(requests):
    return [r.rid for r in requests]


def test_fcfs_admits_in_arrival_order():
    _, sched = make(64)
    for i in [3, 0, 4, 1, 2]:
        sched.add(request(f"r{i}", [i] * 32, float(i)))
    assert rids(sched.schedule(10.0).admitted) == ["r0", "r1", "r2", "r3", "r4"]


def test_lpm_puts_the_cached_request_first_and_fcfs_ignores_the_cache():
    for policy, want in (("lpm", ["hot", "cold"]), ("fcfs", ["cold", "hot"])):
        manager, sched = make(64, policy)
        shared = list(range(64))
        warm(manager, shared)
        sched.add(request("cold", [999] * 80, 0.0))
        sched.add(request("hot", shared + [7] * 16, 1.0))
        plan = sched.schedule(2.0)
        assert rids(plan.admitted) == want
        hot = next(r for r in plan.admitted if r.rid == "hot")
        assert hot.num_cached == 64 and hot.num_computed == 64
        work = next(w for w in plan.work if w.request is hot)
        assert (work.start, work.count, work.emits) == (64, 16, True)


def test_what_happens_when_the_head_does_not_fit():
    """fcfs waits behind it, lpm skips it, lpm_aging skips it until it starves
    (reference: mercury/scheduler.py:155-160)."""
    for policy, want in (("fcfs", []), ("lpm", ["small"]), ("lpm_aging", ["small"])):
        _, sched = make(6, policy, max_wait_s=5.0)
        sched.add(request("big", list(range(160)), 0.0))
        sched.add(request("small", list(range(32)), 1.0))
        assert rids(sched.schedule(2.0).admitted) == want
    _, sched = make(6, "lpm_aging", max_wait_s=5.0)
    sched.add(request("big", list(range(160)), 0.0))
    assert sched.schedule(20.0).admitted == []         # starving: blocks admission, is not skipped
    sched.add(request("small", list(range(32)), 19.0))
    assert sched.schedule(20.0).admitted == []


def test_aging_arithmetic():
    """(reference: tests/test_scheduler.py:85-123)"""
    manager, sched = make(512, "lpm_aging", aging_tokens_per_s=2000.0, max_wait_s=30.0)
    shared = list(range(2048))
    warm(manager, shared)
    cold = request("cold", [99_999] * 80, 0.0)
    assert sched.score(cold, 1.0) < sched.score(request("h1", shared + [7] * 16, 1.0), 1.0)
    assert sched.score(cold, 2.0) > sched.score(request("h2", shared + [7] * 16, 2.0), 2.0)
    hot = request("hot", shared + [7] * 16, 1.0)
    assert all(sched.score(cold, t) < sched.score(hot, t) for t in (2.0, 5.0, 20.0))
    sched.max_wait_s = 5.0
    assert sched.score(cold, 5.0) == float("inf")


def test_scan_limit_bounds_the_scoring():
    _, sched = make(8, "lpm", max_running=1, scan_limit=128)
    for i in range(200):
        sched.add(request(f"r{i}", list(range(32)), float(i)))
    sched.schedule(500.0)
    assert sched.stats["scored_requests"] == 128 and sched.stats["scan_limit_exceeded"] == 1


def test_prompts_are_cut_into_portions_under_the_token_budget():
    _, sched = make(64, prefill_budget=48)
    sched.add(request("a", list(range(100)), 0.0))
    sched.add(request("b", list(range(200, 230)), 1.0))
    seen = []
    for step in range(6):
        plan = sched.schedule(float(step))
        seen.append([(w.request.rid, w.start, w.count, w.emits) for w in plan.work])
        assert plan.num_prefill_tokens <= 48
        finish_step(plan)
    assert seen[0] == [("a", 0, 48, False)]                       # budget spent on a
    assert seen[1] == [("a", 48, 48, False)]
    assert seen[2] == [("a", 96, 4, True), ("b", 0, 30, True)]    # the rest of a, then b fits
    assert seen[3] == [("a", 100, 1, True), ("b", 30, 1, True)]   # both decode
    assert [w.count for w in sched.schedule(9.0).work] == [1, 1]


def test_decoding_goes_on_beside_a_long_prompt():
    _, sched = make(64, prefill_budget=32)
    sched.add(request("short", list(range(8)), 0.0))
    finish_step(sched.schedule(0.0))
    sched.add(request("long", list(range(100, 190)), 1.0))
    for step, want in enumerate([(0, 32), (32, 32), (64, 26)]):
        plan = sched.schedule(1.0 + step)
        assert [(w.request.rid, w.count) for w in plan.work][0] == ("short", 1)
        long_work = plan.work[1]
        assert (long_work.start, long_work.count) == want
        assert long_work.emits == (step == 2)
        assert rids(plan.decode) == ["short"] and (rids(plan.prefill) == ["long"])
        finish_step(plan)


def test_preemption_takes_the_newest_admitted_and_requeues_by_arrival():
    """Four 2-page requests fill an 8-page pool exactly, then each needs a third page
    (reference: tests/test_scheduler.py:147-190)."""
    manager, sched = make(8)
    for i in range(4):
        sched.add(request(f"r{i}", list(range(i * 100, i * 100 + 32)), float(i), max_tokens=64))
    finish_step(sched.schedule(5.0))
    assert manager.num_available() == 0
    plan = sched.schedule(6.0)
    assert rids(plan.preempted) == ["r3", "r2"] and rids(sched.running) == ["r0", "r1"]
    assert rids(w.request for w in plan.work) == ["r0", "r1"]
    victim = plan.preempted[0]
    assert victim.state == RequestState.WAITING and victim.num_computed == 0
    assert victim.preemptions == 1 and not manager.holds("r3")
    assert rids(sched.waiting) == ["r2", "r3"]                    # back in arrival order
    assert len(victim.hashes) == 2                                # rehashed over prompt + output
    manager.check_invariants()


def test_a_preempted_request_starts_over_with_its_output_as_prompt():
    manager, sched = make(5, prefill_budget=64)
    a, b = request("a", list(range(32)), 0.0, 40), request("b", list(range(100, 132)), 1.0, 40)
    sched.add(a)
    sched.add(b)
    finish_step(sched.schedule(0.0))                 # both admitted: 2 + 2 pages, 1 spare
    plan = sched.schedule(1.0)       # a takes the spare page for its token 33; b needs one too
    assert rids(plan.preempted) == ["b"] and b.seq_len == 33 and b.num_computed == 0
    # and is admitted again only when its 3 pages fit
    assert rids(plan.admitted) == []
    finish_step(plan)
    sched.drop(a)
    plan = sched.schedule(3.0)
    assert rids(plan.admitted) == ["b"]
    assert [(w.start, w.count, w.emits) for w in plan.work] == [(0, 33, True)]
    assert b.recomputed_tokens == 32 + 33


def test_windowed_groups_take_pages_portion_by_portion():
    slots = {0: FULL, 1: CacheSpec(2, 16, window=24)}
    manager, sched = make(16, prefill_budget=40, slots=slots)
    sched.add(request("a", list(range(150)), 0.0, max_tokens=4))
    held = []
    for step in range(6):
        plan = sched.schedule(float(step))
        finish_step(plan)
        for w in plan.work:
            manager.trim(w.request.rid, w.request.num_computed)
        pool = manager.groups[1].pool
        held.append(pool.num_pages - pool.num_available())
        manager.check_invariants()
    assert len(manager.table("a", 0)) == 10          # all keys: the whole prompt at admission
    assert max(held) <= 5 and held[-1] <= 3          # the window never holds more than it sees


def test_random_workload_through_the_engine_returns_every_page():
    rng = random.Random(4)
    h = build(policy="fcfs", num_blocks=48, max_running=4, prefill_budget=64, debug_invariants=True)
    for i in range(200):
        prompt = [rng.randrange(50)] * 16 + [rng.randrange(10_000) for _ in range(rng.randrange(1, 80))]
        h.submit(f"r{i}", prompt, max_tokens=rng.randrange(1, 12))
    h.drain()
    assert h.engine.metrics.counters["finished_requests"] == 200
    assert h.engine.leaked_blocks() == 0


def test_preemption_heavy_run_stays_consistent():
    """(reference: tests/test_scheduler.py:205-214)"""
    h = build(num_blocks=20, max_running=8, max_model_len=256, debug_invariants=True)
    for i in range(40):
        h.submit(f"r{i}", list(range(i, i + 64)), max_tokens=40)
    h.drain()
    assert h.engine.metrics.counters["finished_requests"] == 40
    assert h.engine.sched.stats["preemptions"] > 0 and h.engine.leaked_blocks() == 0
    for i in range(40):
        rid = f"r{i}"
        assert h.tokens(rid) == [h.executor.token_for(rid, k) for k in range(40)]


STEP_DT = 0.02


def grouped_stream(policy, groups=6, steps=600, seed=5, **cfg):
    """Several prefix groups whose working set does not fit, arriving interleaved
    (reference: tests/test_scheduler.py:273-287)."""
    rng = random.Random(seed)
    prefixes = [list(range(g * 10_000, g * 10_000 + 128)) for g in range(groups)]
    h = build(policy=policy, num_blocks=28, max_running=4, max_model_len=512, **cfg)
    for step in range(steps):
        if rng.random() < 0.9:
            suffix = [rng.randrange(9_000)] * rng.randrange(8, 32)
            h.submit(f"r{step}", prefixes[rng.randrange(groups)] + suffix, max_tokens=6)
        h.engine.step()
        h.clock.tick(STEP_DT)
    return h


def test_prefix_aware_order_wins_under_pressure_and_the_deadline_bounds_the_wait():
    fcfs = grouped_stream("fcfs").engine.manager.main_pool
    lpm = grouped_stream("lpm").engine.manager.main_pool
    aged = grouped_stream("lpm_aging", max_wait_s=2.0).engine.manager.main_pool
    assert lpm.hit_rate() > fcfs.hit_rate() + 0.05
    assert fcfs.hit_rate() < aged.hit_rate() < lpm.hit_rate()
    assert lpm.stats["evictions"] < fcfs.stats["evictions"]


def test_a_plan_says_when_the_next_one_will_be_the_same_a_token_further():
    """`steady`: every request decodes and none reaches its length with this step's token, and
    nobody waits for a place that is free."""
    _, sched = make(64, max_running=2)
    sched.add(request("a", [1] * 20, 0.0, max_tokens=4))
    sched.add(request("b", [2] * 5, 1.0, max_tokens=6))
    plan = sched.schedule(2.0)
    assert not plan.steady                       # prompts
    finish_step(plan)
    plan = sched.schedule(3.0)
    assert rids(plan.decode) == ["a", "b"] and plan.steady
    sched.add(request("c", [3] * 5, 3.5))
    finish_step(plan)
    plan = sched.schedule(4.0)
    assert plan.steady                           # c waits, but no place is free
    sched.max_running = 3
    finish_step(plan)
    plan = sched.schedule(5.0)
    assert rids(plan.admitted) == ["c"] and not plan.steady
    sched.abort("c")
    # a has 3 of its 4 tokens: this step's token is its last
    assert len(sched.running[0].out) == 3 and not sched.schedule(6.0).steady
