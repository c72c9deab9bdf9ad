from .manager import (CacheFull, CacheGroupSpec, CacheManager, PagePool, StateSpec,
                      kv_cache_budget)

__all__ = ["CacheFull", "CacheGroupSpec", "CacheManager", "PagePool", "StateSpec",
           "kv_cache_budget"]
