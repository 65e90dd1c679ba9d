from .pages import (FREED, CacheError, CacheManager, OutOfPages, OutOfSlots, PagePool, SlotPool, group_needs)
from .storage import CacheStorage, PagedView, StateView

__all__ = ["FREED", "CacheError", "CacheManager", "OutOfPages", "OutOfSlots", "PagePool", "SlotPool", "group_needs",
           "CacheStorage", "PagedView", "StateView"]
