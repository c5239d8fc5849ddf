from .pages import PagePool, PageError
from .manager import CacheManager, CacheLayout, KVView, LayerCache

__all__ = ["PagePool", "PageError", "CacheManager", "CacheLayout", "KVView", "LayerCache"]
