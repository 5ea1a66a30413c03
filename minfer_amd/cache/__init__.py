from .paged import PAGE, Cache, CacheError, CacheFull, KVGroup, KVRequest, PagePool, StateRequest

__all__ = ["PAGE", "Cache", "CacheError", "CacheFull", "KVGroup", "KVRequest", "PagePool", "StateRequest"]
