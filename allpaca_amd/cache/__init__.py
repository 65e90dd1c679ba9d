from .pages import (FREED, CacheError, CacheManager, OutOfPages, OutOfSlots, PagePool, SlotPool, group_needs)
from .storage import CacheStorage, CacheTooLarge, PagedView, StateView
from .estimate import CacheEstimate

__all__ = ["FREED", "CacheError", "CacheManager", "OutOfPages", "OutOfSlots", "PagePool", "SlotPool", "group_needs",
           "CacheStorage", "CacheTooLarge", "PagedView", "StateView", "CacheEstimate"]
