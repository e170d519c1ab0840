"""The cache manager: block tables per request over one page pool per group of cache slots.

Cache slots (one per writing entry of the model's execution list) with the same need (key/
value heads, head size, window) form a *group*.  A group has pages of its own (a
:class:`PagePool`) and every request has one block table per group; all slots of a group use
that table, each over its own key and value tensors.

* A group that keeps **all keys** takes the pages for a whole prompt at admission (with the
  reusable prefix pages first, when prefix sharing is on) and one more page whenever decoding
  crosses a page edge.
* A group with a **window** takes pages step by step, for the tokens of the step, and gives
  back every page whose last position the window has passed; the table keeps -1 there.
* Pages go back to their pool when the request ends, is aborted or is preempted.

Prefix sharing needs every group to keep all keys and no mixer to carry per-request state;
otherwise a cached page does not describe all a later request needs, and admission passes no
hashes.  Beside the pages the manager hands out one state slot per request.
"""

from __future__ import annotations

from dataclasses import dataclass, field

from ..parts.base import CacheSpec
from .pages import PagePool
from .state_slots import StateSlotPool


@dataclass
class CacheGroup:
    spec: CacheSpec
    slots: list            # cache slot ids (execution-list cache ids) that use this group
    pool: PagePool


@dataclass
class RequestPages:
    tables: list                              # per group: list of page ids, -1 = given back
    first_live: list                          # per group: index of the first page still held
    state_slot: int | None = None
    cached_tokens: int = 0
    committed: int = 0                        # full pages already offered to the prefix cache
    extra: dict = field(default_factory=dict)


class CacheManager:
    def __init__(self, cache_slots: dict, num_pages: int, page_size: int, max_requests: int,
                 has_state: bool = False):
        """cache_slots: slot id -> CacheSpec, as the model's execution list declares them."""
        self.page_size = int(page_size)
        self.groups: list = []
        self.group_of_slot: dict = {}
        for slot, spec in sorted(cache_slots.items()):
            for gi, group in enumerate(self.groups):
                if group.spec == spec:
                    group.slots.append(slot)
                    self.group_of_slot[slot] = gi
                    break
            else:
                self.group_of_slot[slot] = len(self.groups)
                self.groups.append(CacheGroup(spec, [slot], PagePool(num_pages, page_size)))
        self.state_slots = StateSlotPool(max_requests)
        self.has_state = bool(has_state)
        self.prefix_sharing = (not has_state) and all(g.spec.window is None for g in self.groups)
        self.requests: dict = {}

    # ---- queries

    @property
    def main_pool(self) -> PagePool | None:
        """The first all-keys group's pool: the one whose hit statistics admission reports."""
        for g in self.groups:
            if g.spec.window is None:
                return g.pool
        return self.groups[0].pool if self.groups else None

    def num_available(self) -> int:
        return min((g.pool.num_available() for g in self.groups), default=0)

    def capacity_tokens(self) -> int:
        return min((g.pool.num_pages for g in self.groups), default=0) * self.page_size

    def cached_prefix_tokens(self, hashes) -> int:
        if not self.prefix_sharing or not self.groups:
            return 0
        return min(len(g.pool.cached_prefix(hashes)) for g in self.groups) * self.page_size

    def table(self, key, group: int) -> list:
        return self.requests[key].tables[group]

    def holds(self, key) -> bool:
        return key in self.requests

    def leaked_pages(self) -> int:
        return sum(g.pool.num_pages - g.pool.num_available() for g in self.groups)

    def _first_needed(self, spec: CacheSpec, next_position: int) -> int:
        """First position a query at `next_position` (and later ones) can still see."""
        return 0 if spec.window is None else max(0, next_position - spec.window + 1)

    # ---- admission, growth, trimming, release

    def admit(self, key, hashes, num_tokens: int):
        """Take a state slot and, in every all-keys group, the pages of a prompt of
        `num_tokens`.  Returns the number of leading tokens whose keys are already cached, or
        None (nothing changed) when it does not fit."""
        if key in self.requests:
            raise AssertionError(f"{key!r} is already admitted")
        if self.state_slots.num_available() == 0:
            return None
        hashes = hashes if self.prefix_sharing else []
        full = [g for g in self.groups if g.spec.window is None]
        hit_pages = None
        if full:
            hit_pages = min(len(g.pool.plan_prompt(hashes, num_tokens)[0]) for g in full)
        done, tables, cached = [], [[] for _ in self.groups], 0
        for gi, g in enumerate(self.groups):
            if g.spec.window is not None:
                continue
            got = g.pool.allocate_prompt(hashes, num_tokens, max_hit=hit_pages)
            if got is None:
                for gj, pages in done:
                    self.groups[gj].pool.release(pages)
                return None
            tables[gi], cached = got[0], got[1]
            done.append((gi, got[0]))
        record = RequestPages(tables=tables, first_live=[0] * len(self.groups),
                              cached_tokens=cached if full else 0)
        record.state_slot = self.state_slots.take(key)
        record.committed = record.cached_tokens // self.page_size
        self.requests[key] = record
        return record.cached_tokens

    def grow(self, key, start: int, new_len: int) -> bool:
        """Make sure every group holds the pages for computing positions [start, new_len).
        Returns False, with nothing changed, when a pool has no page left."""
        record = self.requests[key]
        ps = self.page_size
        want_pages = -(-new_len // ps)
        added = []
        ok = True
        for gi, g in enumerate(self.groups):
            table = record.tables[gi]
            if g.spec.window is not None and len(table) < want_pages:
                # Pages wholly before the window of the first new query are never read.
                skip_to = self._first_needed(g.spec, start) // ps
                while len(table) < min(skip_to, want_pages):
                    table.append(-1)
                record.first_live[gi] = max(record.first_live[gi], min(skip_to, len(table)))
            while len(table) < want_pages:
                page = g.pool.append_page()
                if page is None:
                    ok = False
                    break
                table.append(page)
                added.append((gi, page))
            if not ok:
                break
        if not ok:
            for gi, page in reversed(added):
                self.requests[key].tables[gi].pop()
                self.groups[gi].pool.release([page])
        return ok

    def trim(self, key, num_computed: int) -> int:
        """Give back the pages of window groups that no later query can see, now that
        positions below `num_computed` are computed.  Returns how many pages went back."""
        record = self.requests[key]
        ps, freed = self.page_size, 0
        for gi, g in enumerate(self.groups):
            if g.spec.window is None:
                continue
            table = record.tables[gi]
            keep_from = min(self._first_needed(g.spec, num_computed) // ps, len(table))
            for index in range(record.first_live[gi], keep_from):
                if table[index] >= 0:
                    g.pool.release([table[index]])
                    table[index] = -1
                    freed += 1
            record.first_live[gi] = max(record.first_live[gi], keep_from)
        return freed

    def commit(self, key, hashes, full_pages: int) -> None:
        """Offer the request's pages [committed, full_pages) to the prefix cache under their
        chain hashes (reference: mercury/engine.py:232-241)."""
        record = self.requests[key]
        if not self.prefix_sharing or full_pages <= record.committed:
            return
        for gi, g in enumerate(self.groups):
            table = record.tables[gi]
            for index in range(record.committed, min(full_pages, len(table), len(hashes))):
                g.pool.commit(table[index], hashes[index])
        record.committed = full_pages

    def free(self, key) -> None:
        """Everything the request holds goes back: pages of every group and its state slot."""
        record = self.requests.pop(key)
        for gi, g in enumerate(self.groups):
            g.pool.release([p for p in record.tables[gi] if p >= 0])
        self.state_slots.give(key)

    # ---- checks and reports

    def check_invariants(self) -> None:
        """No page lost, held twice without a shared hash, or freed twice; state slots whole."""
        for gi, g in enumerate(self.groups):
            g.pool.check_invariants()
            held = {}
            for key, record in self.requests.items():
                for page in record.tables[gi]:
                    if page < 0:
                        continue
                    held[page] = held.get(page, 0) + 1
            for page, count in held.items():
                if g.pool.holders[page] != count:
                    raise AssertionError(
                        f"group {gi}: page {page} is in {count} tables but has "
                        f"{g.pool.holders[page]} holders")
                if count > 1 and g.pool.hash_of[page] is None:
                    raise AssertionError(f"group {gi}: unhashed page {page} is shared")
            stray = [p for p in range(g.pool.num_pages) if g.pool.holders[p] and p not in held]
            if stray:
                raise AssertionError(f"group {gi}: pages {stray} are held by no request")
        self.state_slots.check_invariants()

    def snapshot(self) -> dict:
        pool = self.main_pool
        out = pool.snapshot() if pool is not None else {}
        out["groups"] = [
            {"slots": len(g.slots), "kv_heads": g.spec.kv_heads, "head_dim": g.spec.head_dim,
             "window": g.spec.window, "available_blocks": g.pool.num_available()}
            for g in self.groups]
        out["state_slots_free"] = self.state_slots.num_available()
        return out
