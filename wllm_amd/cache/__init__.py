from wllm_amd.cache.manager import CacheManager, CacheNeed, LayerGroup, OutOfSlots, RequestCache
from wllm_amd.cache.pages import OutOfPages, PageAccountingError, PagePool

__all__ = ["CacheManager", "CacheNeed", "LayerGroup", "OutOfSlots", "RequestCache",
           "OutOfPages", "PageAccountingError", "PagePool"]
