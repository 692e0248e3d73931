from .manager import CacheError, CacheManager, KVGroupSpec, OutOfPages, PagePool, StateSpec

__all__ = ["CacheError", "CacheManager", "KVGroupSpec", "OutOfPages", "PagePool", "StateSpec"]
