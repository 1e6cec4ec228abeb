from .allocator import OutOfPages, PagePool
from .manager import CacheManager, PagedGroup, StateSlots, pages_for
from .prefix import PrefixCache

__all__ = ["OutOfPages", "PagePool", "CacheManager", "PagedGroup", "StateSlots", "pages_for", "PrefixCache"]
