from tokenmill_amd.cache.allocator import OutOfPages, PageAllocator, SlotAllocator
from tokenmill_amd.cache.manager import RELEASED, AllocStatus, CacheManager, RequestCache

__all__ = ["OutOfPages", "PageAllocator", "SlotAllocator", "RELEASED", "AllocStatus", "CacheManager", "RequestCache"]
