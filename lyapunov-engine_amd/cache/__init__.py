from .manager import CacheError, CacheManager, CachePools, GroupConfig

__all__ = ["CacheError", "CacheManager", "CachePools", "GroupConfig"]
