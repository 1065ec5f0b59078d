from pyre_amd.cache.allocator import OutOfPages, PageAllocator
from pyre_amd.cache.manager import RELEASED, CacheManager, PageGroup, StateGroup

__all__ = ["OutOfPages", "PageAllocator", "CacheManager", "PageGroup", "StateGroup", "RELEASED"]
