from .manager import (PAGE, CacheError, CacheFull, CacheManager, KvSpec, KvView, PageBook, PagedSpec, PagedView,
                      StateSpec)

__all__ = ["PAGE", "CacheError", "CacheFull", "CacheManager", "KvSpec", "KvView", "PageBook", "PagedSpec", "PagedView",
           "StateSpec"]
