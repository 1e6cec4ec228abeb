from .allocator import PageAllocator
from .manager import CacheManager, PagedGroup, StateSlots, pages_for
from .prefix import PrefixCache

__all__ = ["PageAllocator", "CacheManager", "PagedGroup", "StateSlots", "pages_for", "PrefixCache"]
