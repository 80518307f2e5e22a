from .manager import (CacheError, CacheManager, OutOfPages, OutOfSlots, PageAllocator,
                      PagedLayerView, RequestCache, StateLayerView)
from .specs import FixedState, PagedKV

__all__ = ["CacheError", "CacheManager", "OutOfPages", "OutOfSlots", "PageAllocator",
           "PagedLayerView", "RequestCache", "StateLayerView", "FixedState", "PagedKV"]
