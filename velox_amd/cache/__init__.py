from .allocator import NULL_PAGE, PoolExhausted, PageAllocator  # noqa: F401
from .manager import CacheManager, PagedView, SequenceCache, StateSlots, StateView, pages_that_fit  # noqa: F401
