from .manager import CacheGroup, CacheManager, LayerCacheView, RequestCache
from .pages import CacheExhaustedError, CacheStateError, PagePool

__all__ = ["CacheGroup", "CacheManager", "LayerCacheView", "RequestCache", "CacheExhaustedError",
           "CacheStateError", "PagePool"]
