"""The cache: slots per sequence, key/value pages per group of layers, fixed-size state."""
from .kv import GroupPlan, KVCache, StateNeed
from .pages import PAGE, CacheError, GroupKey, GroupPages, OutOfPages, OutOfSlots, PagePool, SlotTable

__all__ = ["PAGE", "CacheError", "OutOfPages", "OutOfSlots", "PagePool", "SlotTable", "GroupKey",
           "GroupPages", "KVCache", "StateNeed", "GroupPlan"]
