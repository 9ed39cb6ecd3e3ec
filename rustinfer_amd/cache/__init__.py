from .pages import CacheError, OutOfPages, PageAllocator
from .manager import CacheManager, KVCacheView, PageGroup, StateView, pages_for
