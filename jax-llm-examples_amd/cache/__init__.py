from .manager import CacheGroup, CacheManager, CacheView
from .pages import OutOfPages, OutOfSlots, PagePool, SlotPool

__all__ = ["CacheGroup", "CacheManager", "CacheView", "OutOfPages", "OutOfSlots", "PagePool", "SlotPool"]
