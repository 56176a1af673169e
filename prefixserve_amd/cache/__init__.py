from .manager import (BLOCK_SIZE, BlockManager, CacheManager, CoreError, RadixTree, StateSlots, blocks_for)

__all__ = ["BLOCK_SIZE", "BlockManager", "CacheManager", "CoreError", "RadixTree", "StateSlots", "blocks_for"]
