from .manager import CacheConfig, CacheGroup, CacheManager, StateSlotPool
from .pages import NO_PAGE, BlockTable, PageAllocator, PageError, pages_for
