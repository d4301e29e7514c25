from .cache import PAGE, Cache, CacheError, KVGroup, KVView, OutOfPages, PagePool, kv_bytes_per_token, tokens_that_fit

__all__ = ["PAGE", "Cache", "CacheError", "KVGroup", "KVView", "OutOfPages", "PagePool", "kv_bytes_per_token", "tokens_that_fit"]
