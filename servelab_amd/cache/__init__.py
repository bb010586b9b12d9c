from .pages import PageAllocator, SlotAllocator
from .manager import CacheManager, PageGroup, StateGroup, RELEASED
from .pool import CachePool, PageBinding, StateBinding
