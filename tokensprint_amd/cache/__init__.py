from tokensprint_amd.cache.pages import (
    CacheManager, GroupLayout, OutOfPages, OutOfSlots, PagePool, RequestCache, StateSlots,
)
from tokensprint_amd.cache.storage import CacheStorage, LayerCache, group_runs, page_bytes

__all__ = ["CacheManager", "GroupLayout", "OutOfPages", "OutOfSlots", "PagePool",
           "RequestCache", "StateSlots", "CacheStorage", "LayerCache", "group_runs",
           "page_bytes"]
