from .manager import (PAGE, CacheFull, CacheManager, CacheNeed, CacheRecord, GroupLayout, RequestCache,
                      StateNeed)
from .pages import PageError, PagePool

__all__ = ["PAGE", "CacheFull", "CacheManager", "CacheNeed", "CacheRecord", "GroupLayout", "RequestCache",
           "StateNeed", "PageError", "PagePool"]
