from .manager import CacheManager, NO_PAGE, PageGroup
from .needs import CacheNeed, CacheView, FixedState, PagedKV
from .pages import CacheAccountingError, OutOfPages, PagePool, SlotPool

__all__ = ["CacheManager", "NO_PAGE", "PageGroup", "CacheNeed", "CacheView", "FixedState", "PagedKV", "CacheAccountingError",
           "OutOfPages", "PagePool", "SlotPool"]
