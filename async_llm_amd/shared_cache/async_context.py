"""One agent's cache view and write target.

Interface parity with the reference ``AsyncContext`` / ``CacheView``
(``python/minisgl/shared_cache/async_context.py:9-40``).
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import List, Optional

from .shared_block import CacheBlock

# Ordered blocks an agent attends to, read as if concatenated.
CacheView = List[CacheBlock]


@dataclass
class AsyncContext:
    """``cache_view`` is what the agent reads; ``output_block`` is where its
    next token is written.  The write block defaults to the view's last block;
    a write block outside the view is legal (the agent then still attends to
    the token it writes, through the planner's single-slot segment).
    ``next_input_id`` carries the not-yet-stored token across a stream break.
    """

    cache_view: CacheView = field(default_factory=list)
    output_block: CacheBlock = None  # type: ignore[assignment]
    next_input_id: Optional[int] = None

    def __post_init__(self) -> None:
        if self.output_block is not None:
            return
        assert self.cache_view, "AsyncContext needs a cache_view or an explicit output_block"
        self.output_block = self.cache_view[-1]

    @property
    def num_cached_tokens(self) -> int:
        return sum(block.num_tokens for block in self.cache_view)
