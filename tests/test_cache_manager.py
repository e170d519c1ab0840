"""The cache manager: groups with pages of their own, windows that give pages back, state
slots, and no page lost, held twice or freed twice under random orders of requests."""

from __future__ import annotations

import random

import pytest

from mercury_amd.cache import CacheManager, PageHasher, StateSlotPool
from mercury_amd.parts import CacheSpec

PS = 8
FULL = CacheSpec(kv_heads=2, head_dim=16, window=None)
WINDOW = CacheSpec(kv_heads=2, head_dim=16, window=20)
OTHER = CacheSpec(kv_heads=1, head_dim=32, window=None)


def test_slots_with_the_same_need_share_a_group():
    m = CacheManager({0: FULL, 1: WINDOW, 2: FULL, 3: OTHER, 4: WINDOW}, 16, PS, 4)
    assert [g.slots for g in m.groups] == [[0, 2], [1, 4], [3]]
    assert {s: m.group_of(s) for s in range(5)} == {0: 0, 2: 0, 1: 1, 4: 1, 3: 2}
    assert not m.prefix_sharing                       # a window group cannot share prefixes
    assert CacheManager({0: FULL, 1: OTHER}, 16, PS, 4).prefix_sharing
    assert not CacheManager({0: FULL}, 16, PS, 4, has_state=True).prefix_sharing


def test_admission_takes_prompt_pages_in_all_key_groups_only():
    m = CacheManager({0: FULL, 1: WINDOW}, 16, PS, 4)
    assert m.admit("a", [], 30) == 0
    assert len(m.table("a", 0)) == 4 and m.table("a", 1) == []
    assert m.grow("a", 0, 30)
    assert len(m.table("a", 1)) == 4
    m.check_invariants()
    m.free("a")
    assert m.leaked_pages() == 0


def test_window_group_gives_pages_back_once_the_window_has_passed_them():
    m = CacheManager({0: WINDOW}, 16, PS, 4)       # window 20, pages of 8
    m.admit("a", [], 1)
    pool = m.groups[0].pool
    computed = 0
    for portion in (30, 7, 2, 33, 1, 1, 1, 40):
        assert m.grow("a", computed, computed + portion)
        table = m.table("a", 0)
        first_key = max(0, computed - 20 + 1)            # oldest key the first new query sees
        assert all(p >= 0 for p in table[first_key // PS: -(-(computed + portion) // PS)])
        computed += portion
        m.trim("a", computed)
        table = m.table("a", 0)
        keep_from = max(0, computed - 20 + 1) // PS       # next query's oldest key
        assert all(p == -1 for p in table[:keep_from])
        assert all(p >= 0 for p in table[keep_from:])
        assert pool.num_pages - pool.num_available() == len(table) - keep_from <= 4
        m.check_invariants()
    m.free("a")
    assert m.leaked_pages() == 0


def test_a_request_joining_late_skips_pages_before_its_window():
    m = CacheManager({0: FULL, 1: WINDOW}, 32, PS, 4)
    m.admit("a", [], 100)
    assert m.grow("a", 90, 100)                          # e.g. after a long cached prefix
    table = m.table("a", 1)
    assert table[: (90 - 19) // PS] == [-1] * 8 and all(p >= 0 for p in table[8:13])


def test_growth_that_does_not_fit_changes_nothing():
    m = CacheManager({0: FULL, 1: OTHER}, 4, PS, 4)
    m.admit("a", [], 16)
    m.admit("b", [], 16)
    before = [list(m.table("a", g)) for g in range(2)]
    assert not m.grow("a", 16, 17)
    assert [list(m.table("a", g)) for g in range(2)] == before
    m.check_invariants()
    m.free("b")
    assert m.grow("a", 16, 17) and len(m.table("a", 0)) == 3


def test_admission_that_does_not_fit_changes_nothing():
    m = CacheManager({0: FULL, 1: OTHER}, 4, PS, 2)
    assert m.admit("a", [], 33) is None and not m.holds("a")
    assert m.num_available() == 4 and m.state_slots.num_available() == 2
    m.admit("a", [], 8)
    m.admit("b", [], 8)
    assert m.admit("c", [], 8) is None                  # no state slot left
    m.check_invariants()


def test_prefix_pages_are_shared_and_survive_their_first_owner():
    h = PageHasher(PS)
    m = CacheManager({0: FULL, 1: OTHER}, 16, PS, 4)
    tokens = list(range(40))
    hashes = h.hashes(tokens)
    assert m.admit("a", hashes, 40) == 0
    m.commit("a", hashes, 5)
    assert m.admit("b", hashes, 40) == 32               # 4 of 5 pages; one token left to compute
    assert m.table("a", 0)[:4] == m.table("b", 0)[:4] and m.table("a", 0)[4] != m.table("b", 0)[4]
    assert m.table("a", 1)[:4] == m.table("b", 1)[:4]
    m.check_invariants()
    m.free("a")
    m.check_invariants()
    assert m.cached_prefix_tokens(hashes) == 40
    m.free("b")
    assert m.leaked_pages() == 0 and m.cached_prefix_tokens(hashes) == 40


def test_state_slots():
    pool = StateSlotPool(3)
    assert [pool.take(k) for k in "abc"] == [0, 1, 2] and pool.take("d") is None
    pool.give("b")
    assert pool.take("d") == 1 and pool.slot_of("d") == 1
    with pytest.raises(AssertionError):
        pool.take("a")
    with pytest.raises(AssertionError):
        pool.give("zz")
    pool.check_invariants()


@pytest.mark.parametrize("seed", [0, 1, 2])
def test_random_orders_of_requests_lose_nothing(seed):
    rng = random.Random(seed)
    h = PageHasher(PS)
    windowed = seed == 2
    slots = {0: FULL, 1: WINDOW, 2: OTHER} if windowed else {0: FULL, 1: OTHER}
    m = CacheManager(slots, 24, PS, 5)
    prefixes = [[rng.randrange(100) for _ in range(rng.choice([16, 24, 40]))] for _ in range(3)]
    live = {}
    for step in range(3000):
        roll = rng.random()
        if roll < 0.3 and len(live) < 6:
            key = f"r{step}"
            tokens = list(rng.choice(prefixes)) + [rng.randrange(100) for _ in range(rng.randrange(1, 30))]
            cached = m.admit(key, h.hashes(tokens), len(tokens))
            if cached is not None:
                assert cached % PS == 0 and cached < len(tokens)
                live[key] = [tokens, cached]
        elif roll < 0.8 and live:
            key = rng.choice(list(live))
            tokens, done = live[key]
            count = rng.randrange(1, 12)
            if done + count > len(tokens):
                tokens.extend(rng.randrange(100) for _ in range(done + count - len(tokens)))
            if m.grow(key, done, done + count):
                live[key][1] = done + count
                m.commit(key, h.hashes(tokens[: done + count]), (done + count) // PS)
                m.trim(key, done + count)
        elif live:
            m.free(live.popitem()[0] if roll < 0.9 else rng.choice(list(live)))
            live = {k: v for k, v in live.items() if m.holds(k)}
        m.check_invariants()
    for key in list(live):
        m.free(key)
    m.check_invariants()
    assert m.leaked_pages() == 0 and m.state_slots.num_available() == 5
    with pytest.raises(KeyError):
        m.free("r0")                                     # freed twice
