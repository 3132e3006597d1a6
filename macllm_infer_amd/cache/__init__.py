from .manager import CacheManager, EntryCache, KVNeed, PagedGroup, StateNeed
from .pages import BlockTable, CacheExhausted, PagePool, SlotPool

__all__ = ["BlockTable", "CacheExhausted", "CacheManager", "EntryCache", "KVNeed", "PagePool", "PagedGroup",
           "SlotPool", "StateNeed"]
