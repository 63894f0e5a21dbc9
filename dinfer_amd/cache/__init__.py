from .block_pool import BlockPool
from .manager import CacheManager, GroupSpec

__all__ = ["BlockPool", "CacheManager", "GroupSpec"]
