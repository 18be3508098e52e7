from .manager import CacheGroup, CacheLayout, CacheManager, RequestCache, StateGroup
from .state import OutOfStateSlots, StateSlots
from .pages import NO_PAGE, OutOfBlocks, PageAllocator, PageTable, pack_tables

__all__ = [
    "PageAllocator", "OutOfBlocks", "CacheGroup", "CacheLayout", "CacheManager", "RequestCache",
    "StateGroup", "OutOfStateSlots", "StateSlots", "NO_PAGE", "PageTable", "pack_tables",
]
