from .allocator import PageAllocator
from .manager import CacheManager, PagedGroup, StateSlots, pages_for

__all__ = ["PageAllocator", "CacheManager", "PagedGroup", "StateSlots", "pages_for"]
