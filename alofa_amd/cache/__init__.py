from .manager import CacheManager, Group, blocks_for
from .pool import BlockPool

__all__ = ["BlockPool", "CacheManager", "Group", "blocks_for"]
