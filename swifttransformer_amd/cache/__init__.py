from .page_pool import PagePool, OutOfPages
from .manager import CacheManager, CacheGroup, RequestCache, OutOfSlots

__all__ = ["PagePool", "OutOfPages", "CacheManager", "CacheGroup", "RequestCache", "OutOfSlots"]
