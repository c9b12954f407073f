from .allocator import PAGE_TOKENS, FreeList, PageTable, pages_for  # noqa: F401
from .cache import KVGroup, KVView, SequenceCache, StateView  # noqa: F401
