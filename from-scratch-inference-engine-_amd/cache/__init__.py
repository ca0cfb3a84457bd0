"""The cache manager: pages of keys and values with a block table per request, one pool per
group of layers with the same need, and slots for per-request state of fixed size."""

from .allocator import OutOfPages, PageAllocator
from .manager import (CacheManager, NoFreeSlot, PagedNeed, RequestCache, StateNeed)

__all__ = ["CacheManager", "NoFreeSlot", "OutOfPages", "PageAllocator", "PagedNeed",
           "RequestCache", "StateNeed"]
