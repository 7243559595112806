from .manager import CacheManager, NO_PAGE, PageGroup
from .needs import FixedState, PagedKV
from .pages import CacheAccountingError, OutOfPages, PagePool, SlotPool

__all__ = ["CacheManager", "NO_PAGE", "PageGroup", "FixedState", "PagedKV", "CacheAccountingError",
           "OutOfPages", "PagePool", "SlotPool"]
