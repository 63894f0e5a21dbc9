from .manager import CacheManager, GroupSpec

__all__ = ["CacheManager", "GroupSpec"]
