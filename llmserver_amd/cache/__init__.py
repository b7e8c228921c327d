from .manager import CacheGroup, CacheManager, LayerCacheView, RequestCache
from .pages import CacheExhaustedError, CacheStateError, PagePool, PageState

__all__ = ["CacheGroup", "CacheManager", "LayerCacheView", "RequestCache", "CacheExhaustedError",
           "CacheStateError", "PagePool", "PageState"]
