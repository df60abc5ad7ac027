"""Paged key/value cache bookkeeping and per-request state slots."""

from .allocator import BlockAllocator, CacheCapacityError, StateSlotPool
from .manager import NO_PAGE, CacheGroup, CacheManager, RequestCache, plan_groups
from .spec import CacheNeeds, CacheView, FixedState, PagedKV

__all__ = ["BlockAllocator", "CacheCapacityError", "CacheGroup", "CacheManager", "CacheNeeds",
           "CacheView", "FixedState", "NO_PAGE", "PagedKV", "RequestCache", "StateSlotPool",
           "plan_groups"]
