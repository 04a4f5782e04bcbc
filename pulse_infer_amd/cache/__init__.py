from .page_pool import OutOfPages, PageError, PagePool
from .manager import CacheError, CacheGroup, CacheManager, PagedKVSpec, StateSlots, StateSpec

__all__ = ["OutOfPages", "PageError", "PagePool", "CacheError", "CacheGroup", "CacheManager", "PagedKVSpec",
           "StateSlots", "StateSpec"]
