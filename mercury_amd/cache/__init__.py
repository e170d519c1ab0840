"""The cache manager: pages, block tables, groups of layers, prefix hashes, state slots.

All of it lives in the host core (C++: ``csrc/host/page_pool.*``, ``cache_manager.*``,
``hashing.*``); this package gives the classes their Python names.

``PagePool(num_pages, page_size)``
    pages free / held / idle-but-indexed; ``reserve`` (a prompt's pages, reusing an indexed
    prefix, or None with nothing changed), ``take`` (one page), ``publish`` (index a full page
    under its chain hash), ``give_back``, ``check_invariants``.
``CacheManager(cache_slots, num_pages, page_size, max_requests, has_state=False)``
    ``cache_slots`` maps a cache slot id to what it needs (:class:`~mercury_amd.parts.CacheSpec`);
    slots with equal needs share a group, a page pool and the requests' block tables.
    ``admit`` / ``grow`` / ``trim`` / ``commit`` / ``free`` per request key.
``PageHasher(page_size, cryptographic=False)``
    chain hashes of full pages of tokens.
``StateSlotPool(n)``
    slots for per-request state of fixed size.
"""

from ..hostcore import core as _core

CacheGroup = _core.CacheGroup
CacheManager = _core.CacheManager
PageHasher = _core.PageHasher
PagePool = _core.PagePool
PagePoolError = _core.PagePoolError
StateSlotPool = _core.StateSlotPool

__all__ = ["CacheGroup", "CacheManager", "PageHasher", "PagePool", "PagePoolError", "StateSlotPool"]
