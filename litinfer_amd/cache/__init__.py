from .pool import PagePool, PagePoolError
from .manager import CacheFull, CacheManager, CacheView

__all__ = ["PagePool", "PagePoolError", "CacheFull", "CacheManager", "CacheView"]
