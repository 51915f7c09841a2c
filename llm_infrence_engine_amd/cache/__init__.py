from .allocator import NULL_PAGE, OutOfPages, PageAllocator
from .manager import CacheGroup, CacheLayout, CacheManager, GroupKey
from .pools import CachePools

__all__ = ["NULL_PAGE", "OutOfPages", "PageAllocator", "CacheGroup", "CacheLayout", "CacheManager", "GroupKey",
           "CachePools"]
