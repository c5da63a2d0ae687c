from .manager import CacheFull, CacheManager, CacheNeed, GroupLayout, RequestCache, StateNeed
from .pages import PageError, PagePool

__all__ = ["CacheFull", "CacheManager", "CacheNeed", "GroupLayout", "RequestCache", "StateNeed",
           "PageError", "PagePool"]
