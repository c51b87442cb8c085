from .manager import CacheManager, PageGroup, RequestCache, group_name
from .pages import CacheBookkeepingError, OutOfPages, PagePool, StateSlots

__all__ = ["CacheManager", "PageGroup", "RequestCache", "group_name", "CacheBookkeepingError", "OutOfPages",
           "PagePool", "StateSlots"]
