from .manager import (CacheError, CacheManager, OutOfPages, OutOfSlots, PageAllocator,
                      PagedLayerView, RequestCache, StateLayerView)
from .specs import FixedState, PagedKV, PagedSpec, PoolSpec

__all__ = ["CacheError", "CacheManager", "OutOfPages", "OutOfSlots", "PageAllocator",
           "PagedLayerView", "RequestCache", "StateLayerView", "FixedState", "PagedKV",
           "PagedSpec", "PoolSpec"]
