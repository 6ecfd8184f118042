"""MI355X-native cache-view attention: a drop-in for AsyncLLM's
``minisgl.shared_cache`` attention path backed by ``libviewattn.so``."""

from . import native
from .kvcache import MHAKVCache, PageAllocator
from .shared_cache import (
    AsyncContext,
    CacheBlock,
    CacheView,
    PrefillSpec,
    SharedBlock,
    SharedCacheAttention,
    SharedCacheAttnMetadata,
    WorkerGroup,
    apply_rope_correction,
)

ViewAttention = SharedCacheAttention

__all__ = [
    "AsyncContext",
    "CacheBlock",
    "CacheView",
    "MHAKVCache",
    "PageAllocator",
    "PrefillSpec",
    "SharedBlock",
    "SharedCacheAttention",
    "SharedCacheAttnMetadata",
    "ViewAttention",
    "WorkerGroup",
    "apply_rope_correction",
    "native",
]
