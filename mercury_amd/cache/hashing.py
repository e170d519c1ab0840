"""Chain hashes of full pages of tokens, the keys of the prefix cache.

h_i = H(h_{i-1}, tokens of page i), h_{-1} = 0, over full pages only, so a page's hash names
the whole prefix that ends with it (reference: mercury/hashing.py:19-46).  The fast mode is a
keyed 64-bit BLAKE2b digest, the same in every process and run (the reference's default is
Python's per-process ``hash``); the cryptographic mode is SHA-256 cut to 128 bits.
"""

from __future__ import annotations

import hashlib
from array import array
from typing import Sequence


class PageHasher:
    def __init__(self, page_size: int, cryptographic: bool = False):
        self.page_size = int(page_size)
        self.cryptographic = bool(cryptographic)

    def page_hash(self, parent: int, tokens: Sequence[int]) -> int:
        payload = array("q", tokens).tobytes()
        if self.cryptographic:
            digest = hashlib.sha256(parent.to_bytes(16, "little") + payload).digest()[:16]
        else:
            digest = hashlib.blake2b(payload, digest_size=8,
                                     key=parent.to_bytes(8, "little")).digest()
        return int.from_bytes(digest, "little")

    def hashes(self, tokens: Sequence[int], parent: int = 0) -> list:
        """One hash per full page of `tokens`."""
        ps, out = self.page_size, []
        for start in range(0, len(tokens) - ps + 1, ps):
            parent = self.page_hash(parent, tokens[start:start + ps])
            out.append(parent)
        return out

    def extend(self, hashes: list, tokens: Sequence[int]) -> int:
        """Grow `hashes` in place to cover every full page of `tokens`; returns pages added."""
        ps = self.page_size
        full = len(tokens) // ps
        parent = hashes[-1] if hashes else 0
        added = 0
        for index in range(len(hashes), full):
            parent = self.page_hash(parent, tokens[index * ps:(index + 1) * ps])
            hashes.append(parent)
            added += 1
        return added
