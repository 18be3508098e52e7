from .allocator import BlockAllocator, OutOfBlocks
from .manager import CacheGroup, CacheLayout, CacheManager, RequestCache, StateGroup
from .state import OutOfStateSlots, StateSlots
from .table import NO_BLOCK, BlockTable, pack_tables

__all__ = [
    "BlockAllocator", "OutOfBlocks", "CacheGroup", "CacheLayout", "CacheManager", "RequestCache",
    "StateGroup", "OutOfStateSlots", "StateSlots", "NO_BLOCK", "BlockTable", "pack_tables",
]
