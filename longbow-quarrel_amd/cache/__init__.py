"""The cache: slots, paged keys and values per layer group, fixed-size state."""
from .manager import CacheGroup, CacheManager, KVGroup, StateGroup, blocks_for
from .slots import BLOCK_SIZE, CacheFull, FreeList

__all__ = ["CacheGroup", "CacheManager", "KVGroup", "StateGroup", "blocks_for", "BLOCK_SIZE", "CacheFull", "FreeList"]
