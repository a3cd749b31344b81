from .allocator import (AllocError, DoubleFree, NotFull, PageAllocator, Release, UnknownPage, pages_for_len,
                        prefix_page_hash)
from .manager import CacheGroup, CacheManager, OutOfPages, RequestCache, plan_groups
from .pools import CachePools

__all__ = ["AllocError", "DoubleFree", "NotFull", "PageAllocator", "Release", "UnknownPage", "pages_for_len",
           "prefix_page_hash", "CacheGroup", "CacheManager", "OutOfPages", "RequestCache", "plan_groups",
           "CachePools"]
