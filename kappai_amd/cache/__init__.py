from .manager import (BundleView, CacheError, CacheManager, OutOfPages, OutOfSlots, PageAllocator,
                      PagedLayerView, RequestCache, StateLayerView)
from .specs import CacheBundle, FixedState, PagedKV, PagedSpec, PoolSpec

__all__ = ["BundleView", "CacheBundle", "CacheError", "CacheManager", "OutOfPages", "OutOfSlots", "PageAllocator",
           "PagedLayerView", "RequestCache", "StateLayerView", "FixedState", "PagedKV",
           "PagedSpec", "PoolSpec"]
