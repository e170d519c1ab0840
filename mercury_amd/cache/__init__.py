"""The cache manager: pages, block tables, groups of layers, prefix hashes, state slots."""

from .hashing import PageHasher
from .manager import CacheGroup, CacheManager
from .pages import PagePool, PagePoolError
from .state_slots import StateSlotPool

__all__ = ["CacheGroup", "CacheManager", "PageHasher", "PagePool", "PagePoolError", "StateSlotPool"]
