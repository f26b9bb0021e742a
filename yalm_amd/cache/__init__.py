from .manager import (PAGE, CacheError, CacheFull, CacheManager, KVGroup, KVRequest, PagePool, SlotAllocator,
                      StateGroup, StateRequest, pages_for)

__all__ = ["PAGE", "CacheError", "CacheFull", "CacheManager", "KVGroup", "KVRequest", "PagePool", "SlotAllocator",
           "StateGroup", "StateRequest", "pages_for"]
