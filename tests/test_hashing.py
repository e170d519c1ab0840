"""Chain hashes of full pages (behaviour of reference tests/test_hashing.py:14-73)."""

from __future__ import annotations

import random

from mercury_amd.cache import PageHasher


def test_only_full_pages_are_hashed():
    h = PageHasher(16)
    assert [len(h.hashes(list(range(n)))) for n in (15, 16, 31, 32)] == [0, 1, 1, 2]


def test_chain_depends_on_every_earlier_token_and_on_nothing_later():
    h = PageHasher(16)
    a, b, c = list(range(64)), list(range(64)), list(range(64))
    b[0], c[63] = 999, -1 & 0x7FFFFFFF
    ha, hb, hc = h.hashes(a), h.hashes(b), h.hashes(c)
    assert all(x != y for x, y in zip(ha, hb))
    assert ha[:3] == hc[:3] and ha[3] != hc[3]


def test_shared_prefix_shares_exactly_the_shared_pages():
    h = PageHasher(16)
    shared = list(range(48))
    left, right = h.hashes(shared + [1] * 16), h.hashes(shared + [2] * 16)
    assert left[:3] == right[:3] and left[3] != right[3]


def test_extend_matches_a_full_recompute_and_counts():
    h = PageHasher(16)
    rng = random.Random(7)
    tokens = [rng.randrange(1000) for _ in range(200)]
    grown: list = []
    for end in range(0, 201, 8):
        h.extend(grown, tokens[:end])
    assert grown == h.hashes(tokens)
    out: list = []
    assert [h.extend(out, tokens[:16]), h.extend(out, tokens[:16]), h.extend(out, tokens[:48])] == [1, 0, 2]


def test_hashes_are_the_same_in_every_process_and_differ_by_mode():
    tokens = list(range(32))
    fast, strong = PageHasher(16), PageHasher(16, cryptographic=True)
    assert fast.hashes(tokens) == PageHasher(16).hashes(tokens)
    assert fast.hashes(tokens)[0] == 0xD85847B14FA46C4   # not Python's per-process hash()
    assert strong.hashes(tokens) != fast.hashes(tokens)
    assert all(0 <= x < 2**128 for x in strong.hashes(tokens))
    assert strong.page_hash(strong.hashes(tokens)[0], tokens[16:32]) == strong.hashes(tokens)[1]
