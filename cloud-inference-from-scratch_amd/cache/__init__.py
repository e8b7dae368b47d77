from .allocator import CacheCapacityFull, DoubleFreeError, PageAllocator
from .manager import PREFIX_HOLDER, CacheManager, CacheStats, FixedState, PagedKV

__all__ = [
    "CacheCapacityFull", "CacheManager", "CacheStats", "DoubleFreeError", "FixedState",
    "PREFIX_HOLDER", "PageAllocator", "PagedKV",
]
