from .mha_pool import MHAKVCache
from .page_allocator import PageAllocator

__all__ = ["MHAKVCache", "PageAllocator"]
