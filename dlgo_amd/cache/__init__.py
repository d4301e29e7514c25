from .cache import PAGE, Cache, CacheError, KVGroup, KVView, OutOfPages, PagePool

__all__ = ["PAGE", "Cache", "CacheError", "KVGroup", "KVView", "OutOfPages", "PagePool"]
