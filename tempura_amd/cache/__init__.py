from .manager import CacheManager, PagesExhausted
from .pools import CachePools, LayerCache
from .rules import VisibilityRule, register_rule

__all__ = ["PagesExhausted", "CacheManager", "CachePools", "LayerCache", "VisibilityRule", "register_rule"]
