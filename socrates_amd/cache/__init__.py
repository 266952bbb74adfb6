from .allocator import NULL_PAGE, BlockAllocator, OutOfBlocks, blocks_for
from .manager import CacheManager, PagedGroup, PagedSlot, RowScalars, StateSlot

__all__ = ["NULL_PAGE", "BlockAllocator", "OutOfBlocks", "blocks_for", "CacheManager",
           "PagedGroup", "PagedSlot", "RowScalars", "StateSlot"]
