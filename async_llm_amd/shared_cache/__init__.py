from .async_context import AsyncContext, CacheView
from .attention import PrefillSpec, SharedCacheAttention, SharedCacheAttnMetadata
from .attention_metadata import page_numbers, upload_page_indices
from .block_ops import BlockKVOps
from .rope_correction import apply_rope_correction
from .shared_block import CacheBlock, SharedBlock
from .worker_group import WorkerGroup

__all__ = [
    "AsyncContext",
    "BlockKVOps",
    "CacheBlock",
    "CacheView",
    "PrefillSpec",
    "SharedBlock",
    "SharedCacheAttention",
    "SharedCacheAttnMetadata",
    "WorkerGroup",
    "apply_rope_correction",
    "page_numbers",
    "upload_page_indices",
]
