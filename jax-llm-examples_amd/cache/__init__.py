from .manager import CacheGroup, CacheManager, CacheView, plan_groups, pool_sizes, tokens_held_at_most
from .pages import OutOfPages, OutOfSlots, PagePool, SlotPool

__all__ = ["CacheGroup", "CacheManager", "CacheView", "OutOfPages", "OutOfSlots", "PagePool", "SlotPool",
           "plan_groups", "pool_sizes", "tokens_held_at_most"]
