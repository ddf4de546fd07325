from wllm_amd.cache.manager import CacheManager, CacheNeed, LayerGroup, OutOfSlots, PagedNeed, RequestCache, StateNeed
from wllm_amd.cache.pages import OutOfPages, PageAccountingError, PagePool

__all__ = ["CacheManager", "CacheNeed", "LayerGroup", "OutOfSlots", "PagedNeed", "RequestCache", "StateNeed",
           "OutOfPages", "PageAccountingError", "PagePool"]
