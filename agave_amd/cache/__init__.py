"""The cache: slots per sequence, key/value pages per group of layers, fixed-size state."""
from .kv import GroupPlan, KVCache, StateNeed
from .pages import PAGE, CacheError, GroupKey, GroupPages, OutOfPages, OutOfSlots, PagePool, SlotTable, pages_in_reach, pool_pages

__all__ = ["PAGE", "CacheError", "OutOfPages", "OutOfSlots", "PagePool", "SlotTable", "GroupKey",
           "GroupPages", "pages_in_reach", "pool_pages", "KVCache", "StateNeed", "GroupPlan"]
