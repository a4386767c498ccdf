from .manager import ABSENT, CacheManager, PageGroup, RunNeed
from .pages import PageAllocator

__all__ = ["ABSENT", "CacheManager", "PageGroup", "RunNeed", "PageAllocator"]
