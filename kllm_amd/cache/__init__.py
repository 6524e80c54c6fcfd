from .pages import CacheError, OutOfPages, PagePool, SlotPool
from .manager import FREED, CacheManager, GroupSpec, RequestCache

__all__ = ["CacheError", "OutOfPages", "PagePool", "SlotPool", "FREED", "CacheManager",
           "GroupSpec", "RequestCache"]
