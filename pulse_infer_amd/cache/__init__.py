from .page_pool import OutOfPages, PageError, PagePool
from .specs import PagedCacheView, PagedKVSpec, StateSpec, StateView
from .manager import CacheError, CacheGroup, CacheManager, StateSlots

__all__ = ["OutOfPages", "PageError", "PagePool", "CacheError", "CacheGroup", "CacheManager", "PagedKVSpec",
           "StateSlots", "StateSpec", "PagedCacheView", "StateView"]
