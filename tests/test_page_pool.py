"""The page pool (host core, C++): the vectors of reference tests/test_allocator.py:27-204
against it, plus what its own design adds (queues as intrusive lists, an audit)."""

from __future__ import annotations

import random

import pytest

from mercury_amd.cache import PageHasher, PagePool, PagePoolError

PS = 16
H = PageHasher(PS)


def filled(pool, tokens):
    hashes = H.hashes(tokens)
    pages, cached = pool.reserve(hashes, len(tokens))
    for i in range(len(tokens) // PS):
        pool.publish(pages[i], hashes[i])
    return pages, cached


def test_starts_empty_and_gets_everything_back():
    pool = PagePool(8, PS)
    pages, cached = filled(pool, list(range(64)))
    assert (cached, len(pages), pool.num_available()) == (0, 4, 4)
    pool.give_back(pages)
    assert pool.num_available() == 8
    pool.check_invariants()


def test_partial_last_page_counts_but_is_not_shared():
    pool = PagePool(8, PS)
    pages, _ = filled(pool, list(range(40)))
    assert len(pages) == 3 and pool.hash_of(pages[2]) is None
    pool.give_back(pages)
    assert (len(pool.idle), len(pool.free)) == (2, 6)


def test_second_identical_prompt_hits():
    pool = PagePool(16, PS)
    first, _ = filled(pool, list(range(80)))
    pool.give_back(first)
    second, cached = filled(pool, list(range(80)))
    assert cached == 64 and second[:4] == first[:4] and second[4] != first[4]
    assert pool.stats["query_tokens"] == 160 and pool.hit_rate() == pytest.approx(0.4)


def test_one_token_is_always_left_to_compute():
    pool = PagePool(16, PS)
    first, _ = filled(pool, list(range(64)))
    pool.give_back(first)
    assert pool.reusable(H.hashes(list(range(64))), 64) == 3        # so one page is new
    assert pool.reusable(H.hashes(list(range(64))), 64, cap=1) == 1
    assert pool.reusable(H.hashes(list(range(64))), 65) == 4


def test_prefix_match_stops_at_the_first_miss():
    pool = PagePool(32, PS)
    left, _ = filled(pool, list(range(64)) + [1] * 16)
    pool.give_back(left)
    assert len(pool.match(H.hashes(list(range(64)) + [2] * 16))) == 4


def test_release_queues_the_tail_for_eviction_before_the_head():
    pool = PagePool(8, PS)
    pages, _ = filled(pool, list(range(128)))
    pool.give_back(pages)
    assert pool.idle == list(reversed(pages))
    assert pool.take() == pages[-1]


def test_failed_allocation_changes_nothing():
    pool = PagePool(4, PS)
    before = pool.snapshot()
    assert pool.reserve([], 128) is None
    after = pool.snapshot()
    assert after["free_blocks"] == before["free_blocks"] and after["query_tokens"] == 0
    assert after["allocation_failures"] == 1
    pool.check_invariants()


def test_pinning_cached_pages_counts_against_capacity():
    pool = PagePool(5, PS)
    first, _ = filled(pool, list(range(64)))
    pool.give_back(first)
    assert pool.reserve(H.hashes(list(range(64)) + [9] * 16), 80) is not None
    assert pool.num_available() == 0


def test_eviction_takes_the_least_recently_released():
    pool = PagePool(4, PS)
    a, _ = filled(pool, list(range(32)))
    pool.give_back(a)
    b, _ = filled(pool, list(range(100, 132)))
    pool.give_back(b)
    fresh, cached = filled(pool, list(range(200, 264)))
    assert cached == 0 and pool.stats["evictions"] == 4 and set(fresh) == set(a) | set(b)


def test_duplicate_content_keeps_the_first_page():
    pool = PagePool(16, PS)
    hashes = H.hashes(list(range(32)))
    left, _ = pool.reserve(hashes, 32)
    right, _ = pool.reserve(hashes, 32)
    pool.publish(left[0], hashes[0])
    pool.publish(right[0], hashes[0])
    assert pool.page_for(hashes[0]) == left[0] and pool.hash_of(right[0]) is None
    pool.give_back(right)
    assert right[0] in pool.free


def test_append_fails_cleanly_when_full_and_double_free_is_caught():
    pool = PagePool(2, PS)
    pages, _ = pool.reserve([], 32)
    assert pool.take() is None
    pool.give_back(pages)
    with pytest.raises(PagePoolError, match="nobody holds"):
        pool.give_back(pages[:1])


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
            got = pool.reserve(hashes, len(tokens))
            if got is not None:
                for i in range(min(len(tokens) // PS, len(got[0]))):
                    pool.publish(got[0][i], hashes[i])
                live.append(got[0])
        elif roll < 0.8:
            pool.give_back(live.pop(rng.randrange(len(live))))
        else:
            page = pool.take()
            if page is not None:
                live.append([page])
        pool.check_invariants()
    for pages in live:
        pool.give_back(pages)
    pool.check_invariants()
    assert pool.num_available() == 64 and sum(pool.holders) == 0
