from .pages import PagePool, PagesExhausted
from .manager import CacheManager
from .pools import CachePools, LayerCache

__all__ = ["PagePool", "PagesExhausted", "CacheManager", "CachePools", "LayerCache"]
