from .pool import PagePool, PagePoolError
from .manager import CacheFull, CacheManager, CacheView, group_needs

__all__ = ["PagePool", "PagePoolError", "CacheFull", "CacheManager", "CacheView", "group_needs"]
