from .pages import NO_PAGE, CacheError, CacheManager, GroupSpec, PagePool, RequestPages, SlotPool
from .storage import CacheStorage, LayerCache

__all__ = ["NO_PAGE", "CacheError", "CacheManager", "GroupSpec", "PagePool", "RequestPages", "SlotPool",
           "CacheStorage", "LayerCache"]
