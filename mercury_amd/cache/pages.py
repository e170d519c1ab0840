"""A pool of fixed-size cache pages with a hash-addressed store of reusable prefix pages.

Every page is in exactly one of three states (reference: mercury/allocator.py:7-16):

    free      no holder, no hash, in the free queue
    in use    held by at least one request's block table
    cached    no holder, hashed, in the eviction queue (oldest release first)

A page id addresses the same page in the keys and the values of every cache slot of the
pool's group.  Pages are not cleared when they change hands; the kernels never read past a
sequence's own length.
"""

from __future__ import annotations

from collections import OrderedDict, deque
from typing import Sequence


class PagePoolError(AssertionError):
    pass


class PagePool:
    def __init__(self, num_pages: int, page_size: int):
        if num_pages <= 0:
            raise ValueError("num_pages must be positive")
        self.num_pages, self.page_size = int(num_pages), int(page_size)
        self.holders = [0] * num_pages
        self.hash_of: list = [None] * num_pages
        self.by_hash: dict = {}
        self.free = deque(range(num_pages))
        self.evictable: OrderedDict = OrderedDict()
        self.stats = {"hit_tokens": 0, "query_tokens": 0, "evictions": 0, "prefills": 0,
                      "allocation_failures": 0}

    # ---- queries

    def num_available(self) -> int:
        return len(self.free) + len(self.evictable)

    def num_cached_pages(self) -> int:
        return len(self.by_hash)

    def hit_rate(self) -> float:
        asked = self.stats["query_tokens"]
        return self.stats["hit_tokens"] / asked if asked else 0.0

    def cached_prefix(self, hashes: Sequence[int]) -> list:
        """Pages holding the longest cached prefix of the hash chain."""
        pages = []
        for h in hashes:
            page = self.by_hash.get(h)
            if page is None:
                break
            pages.append(page)
        return pages

    def plan_prompt(self, hashes: Sequence[int], num_tokens: int, max_hit: int | None = None):
        """(cached pages a prompt would reuse, new pages it needs); changes nothing.  One
        token is always left to compute, or the prompt would yield no logits
        (reference: mercury/allocator.py:64-73)."""
        ps = self.page_size
        limit = (num_tokens - 1) // ps
        if max_hit is not None:
            limit = min(limit, max_hit)
        hit = self.cached_prefix(hashes)[:limit]
        return hit, -(-num_tokens // ps) - len(hit)

    # ---- changes

    def _take(self) -> int:
        if self.free:
            return self.free.popleft()
        page, _ = self.evictable.popitem(last=False)
        del self.by_hash[self.hash_of[page]]
        self.hash_of[page] = None
        self.stats["evictions"] += 1
        return page

    def allocate_prompt(self, hashes: Sequence[int], num_tokens: int, max_hit: int | None = None):
        """(pages, cached token count), or None with nothing changed when it does not fit
        (reference: mercury/allocator.py:75-95)."""
        hit, need = self.plan_prompt(hashes, num_tokens, max_hit)
        pinned = sum(1 for p in hit if self.holders[p] == 0)
        if need > self.num_available() - pinned:
            self.stats["allocation_failures"] += 1
            return None
        for p in hit:
            if self.holders[p] == 0:
                del self.evictable[p]
            self.holders[p] += 1
        fresh = [self._take() for _ in range(need)]
        for p in fresh:
            self.holders[p] = 1
        cached = len(hit) * self.page_size
        self.stats["hit_tokens"] += cached
        self.stats["query_tokens"] += num_tokens
        self.stats["prefills"] += 1
        return hit + fresh, cached

    def append_page(self):
        if self.num_available() == 0:
            return None
        page = self._take()
        self.holders[page] = 1
        return page

    def commit(self, page: int, h: int) -> None:
        """Make a full page findable by its hash; the first page with a hash keeps it
        (reference: mercury/allocator.py:104-108)."""
        if self.hash_of[page] is None and h not in self.by_hash:
            self.hash_of[page] = h
            self.by_hash[h] = page

    def release(self, pages: Sequence[int]) -> None:
        """Give pages back, last first, so that a request's private tail is evicted before
        the prefix others may share (reference: mercury/allocator.py:110-121)."""
        for p in reversed(pages):
            if self.holders[p] <= 0:
                raise PagePoolError(f"page {p} is given back but nobody holds it")
            self.holders[p] -= 1
            if self.holders[p] == 0:
                if self.hash_of[p] is not None:
                    self.evictable[p] = None
                else:
                    self.free.append(p)

    def reset_stats(self) -> None:
        for key in self.stats:
            self.stats[key] = 0

    def snapshot(self) -> dict:
        return {
            "num_blocks": self.num_pages,
            "block_size": self.page_size,
            "free_blocks": len(self.free),
            "evictable_blocks": len(self.evictable),
            "available_blocks": self.num_available(),
            "cached_blocks": self.num_cached_pages(),
            "hit_rate": self.hit_rate(),
            **self.stats,
        }

    def check_invariants(self) -> None:
        """Every page in exactly one state; the hash maps agree.  O(pages)."""
        free, evictable = set(self.free), set(self.evictable)
        if len(free) != len(self.free):
            raise PagePoolError("a page is in the free queue twice")
        if free & evictable:
            raise PagePoolError(f"pages both free and cached: {sorted(free & evictable)}")
        for p in range(self.num_pages):
            held, hashed = self.holders[p], self.hash_of[p] is not None
            if held < 0:
                raise PagePoolError(f"page {p} has {held} holders")
            if p in free:
                if held or hashed:
                    raise PagePoolError(f"free page {p} is held or hashed")
            elif p in evictable:
                if held or not hashed:
                    raise PagePoolError(f"cached page {p} is held or has no hash")
            elif held == 0:
                raise PagePoolError(f"page {p} has no holder but is in no queue")
        for h, p in self.by_hash.items():
            if self.hash_of[p] != h:
                raise PagePoolError(f"hash {h} maps to page {p}, whose hash is {self.hash_of[p]}")
