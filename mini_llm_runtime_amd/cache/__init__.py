"""Paged keys and values, block tables, and per-request state slots."""

from .block_pool import BlockAllocator, BlockPoolExhaustedError, SlotPool, blocks_for
from .manager import CacheManager, CacheStats, KVGroup, RequestCache, StepLayout, VisibilityError
from .spec import PagedKVSpec, PagedSpec, SiteCacheSpec, SlotSpec, SlotStateSpec
from .views import KVView, StateView

__all__ = [
    "BlockAllocator",
    "BlockPoolExhaustedError",
    "CacheManager",
    "CacheStats",
    "KVGroup",
    "KVView",
    "PagedKVSpec",
    "PagedSpec",
    "SiteCacheSpec",
    "SlotSpec",
    "StateView",
    "RequestCache",
    "SlotPool",
    "SlotStateSpec",
    "StepLayout",
    "VisibilityError",
    "blocks_for",
]
