from .manager import CacheGroup, CacheManager
from .pages import OutOfPages, PageAllocator

__all__ = ["CacheGroup", "CacheManager", "OutOfPages", "PageAllocator"]
