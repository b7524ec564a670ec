from .manager import (CacheError, CacheFull, CacheManager, KvSpec, KvView, PageBook, StateSpec)

__all__ = ["CacheError", "CacheFull", "CacheManager", "KvSpec", "KvView", "PageBook", "StateSpec"]
