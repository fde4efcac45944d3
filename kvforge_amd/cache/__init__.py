from kvforge_amd.cache.block_pool import BlockPool, NoFreeBlocksError
from kvforge_amd.cache.manager import RELEASED, CacheGroup, CacheManager, CacheStats, StateSlots

__all__ = ["BlockPool", "NoFreeBlocksError", "RELEASED", "CacheGroup", "CacheManager",
           "CacheStats", "StateSlots"]
