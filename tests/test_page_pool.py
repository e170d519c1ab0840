"""The page pool: vectors of reference tests/test_allocator.py:27-204 against our pool."""

from __future__ import annotations

import random

import pytest

from mercury_amd.cache import PageHasher, PagePool, PagePoolError

PS = 16
H = PageHasher(PS)


def filled(pool, tokens):
    hashes = H.hashes(tokens)
    pages, cached = pool.allocate_prompt(hashes, len(tokens))
    for i in range(len(tokens) // PS):
        pool.commit(pages[i], hashes[i])
    return pages, cached


def test_starts_empty_and_gets_everything_back():
    pool = PagePool(8, PS)
    pages, cached = filled(pool, list(range(64)))
    assert (cached, len(pages), pool.num_available()) == (0, 4, 4)
    pool.release(pages)
    assert pool.num_available() == 8
    pool.check_invariants()


def test_partial_last_page_counts_but_is_not_shared():
    pool = PagePool(8, PS)
    pages, _ = filled(pool, list(range(40)))
    assert len(pages) == 3 and pool.hash_of[pages[2]] is None
    pool.release(pages)
    assert (len(pool.evictable), len(pool.free)) == (2, 6)


def test_second_identical_prompt_hits():
    pool = PagePool(16, PS)
    first, _ = filled(pool, list(range(80)))
    pool.release(first)
    second, cached = filled(pool, list(range(80)))
    assert cached == 64 and second[:4] == first[:4] and second[4] != first[4]
    assert pool.stats["query_tokens"] == 160 and pool.hit_rate() == pytest.approx(0.4)


def test_one_token_is_always_left_to_compute():
    pool = PagePool(16, PS)
    first, _ = filled(pool, list(range(64)))
    pool.release(first)
    hit, need = pool.plan_prompt(H.hashes(list(range(64))), 64)
    assert (len(hit), need) == (3, 1)
    assert pool.plan_prompt(H.hashes(list(range(64))), 64, max_hit=1)[1] == 3


def test_prefix_match_stops_at_the_first_miss():
    pool = PagePool(32, PS)
    left, _ = filled(pool, list(range(64)) + [1] * 16)
    pool.release(left)
    assert len(pool.cached_prefix(H.hashes(list(range(64)) + [2] * 16))) == 4


def test_release_queues_the_tail_for_eviction_before_the_head():
    pool = PagePool(8, PS)
    pages, _ = filled(pool, list(range(128)))
    pool.release(pages)
    assert list(pool.evictable) == list(reversed(pages))
    assert pool._take() == pages[-1]


def test_failed_allocation_changes_nothing():
    pool = PagePool(4, PS)
    before = pool.snapshot()
    assert pool.allocate_prompt([], 128) is None
    after = pool.snapshot()
    assert after["free_blocks"] == before["free_blocks"] and after["query_tokens"] == 0
    assert after["allocation_failures"] == 1
    pool.check_invariants()


def test_pinning_cached_pages_counts_against_capacity():
    pool = PagePool(5, PS)
    first, _ = filled(pool, list(range(64)))
    pool.release(first)
    assert pool.allocate_prompt(H.hashes(list(range(64)) + [9] * 16), 80) is not None
    assert pool.num_available() == 0


def test_eviction_takes_the_least_recently_released():
    pool = PagePool(4, PS)
    a, _ = filled(pool, list(range(32)))
    pool.release(a)
    b, _ = filled(pool, list(range(100, 132)))
    pool.release(b)
    fresh, cached = filled(pool, list(range(200, 264)))
    assert cached == 0 and pool.stats["evictions"] == 4 and set(fresh) == set(a) | set(b)


def test_duplicate_content_keeps_the_first_page():
    pool = PagePool(16, PS)
    hashes = H.hashes(list(range(32)))
    left, _ = pool.allocate_prompt(hashes, 32)
    right, _ = pool.allocate_prompt(hashes, 32)
    pool.commit(left[0], hashes[0])
    pool.commit(right[0], hashes[0])
    assert pool.by_hash[hashes[0]] == left[0] and pool.hash_of[right[0]] is None
    pool.release(right)
    assert right[0] in pool.free


def test_append_fails_cleanly_when_full_and_double_free_is_caught():
    pool = PagePool(2, PS)
    pages, _ = pool.allocate_prompt([], 32)
    assert pool.append_page() is None
    pool.release(pages)
    with pytest.raises(PagePoolError, match="nobody holds"):
        pool.release(pages[:1])


def test_random_churn_keeps_every_invariant():
    rng = random.Random(1234)
    pool = PagePool(64, PS)
    prefixes = [[rng.randrange(5000) for _ in range(rng.choice([32, 64, 96]))] for _ in range(6)]
    live = []
    for _ in range(4000):
        roll = rng.random()
        if roll < 0.5 or not live:
            tokens = list(rng.choice(prefixes)) + [rng.randrange(5000) for _ in range(rng.randrange(1, 40))]
            hashes = H.hashes(tokens)
            got = pool.allocate_prompt(hashes, len(tokens))
            if got is not None:
                for i in range(min(len(tokens) // PS, len(got[0]))):
                    pool.commit(got[0][i], hashes[i])
                live.append(got[0])
        elif roll < 0.8:
            pool.release(live.pop(rng.randrange(len(live))))
        else:
            page = pool.append_page()
            if page is not None:
                live.append([page])
        pool.check_invariants()
    for pages in live:
        pool.release(pages)
    pool.check_invariants()
    assert pool.num_available() == 64 and sum(pool.holders) == 0
