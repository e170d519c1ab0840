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
    assert fast.hashes(tokens)[0] == 16304858532140510287   # not Python's per-process hash()
    assert strong.hashes(tokens) != fast.hashes(tokens)
    assert all(0 <= x < 2**128 for x in strong.hashes(tokens))
    assert strong.page_hash(strong.hashes(tokens)[0], tokens[16:32]) == strong.hashes(tokens)[1]


def test_the_strong_mode_is_sha256_of_parent_and_tokens():
    """The host core's own SHA-256 against hashlib's: the published vector for "abc", and a
    page hash recomputed here from its definition (parent as 16 bytes, tokens as 8-byte
    integers, little-endian; the first 128 bits of the digest, little-endian)."""
    import hashlib
    from array import array

    from mercury_amd.hostcore import core

    assert core.sha256(b"abc").hex() == \
        "ba7816bf8f01cfea414140de5dae2223b00361a396177a9cb410ff61f20015ad"
    for size in (0, 55, 56, 63, 64, 65, 200):
        data = bytes(range(256))[:size] if size <= 256 else b""
        assert core.sha256(data) == hashlib.sha256(data).digest()
    strong = PageHasher(16, cryptographic=True)
    tokens = [7, 0, 2**31 - 1] + list(range(13))
    parent = 0
    for _ in range(2):
        payload = parent.to_bytes(16, "little") + array("q", tokens).tobytes()
        want = int.from_bytes(hashlib.sha256(payload).digest()[:16], "little")
        assert strong.page_hash(parent, tokens) == want
        parent = want
