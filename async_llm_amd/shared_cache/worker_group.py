"""The set of agents decoded together in one step.

Interface parity with the reference ``WorkerGroup``
(``python/minisgl/shared_cache/worker_group.py:9-97``): positional list of
``AsyncContext`` or the keyword form ``cache_structure=..., write_to=...``;
at most one writer per block per step.
"""

from __future__ import annotations

from typing import Iterator, List, Optional, Sequence, Union

from .async_context import AsyncContext
from .shared_block import CacheBlock


class WorkerGroup:
    def __init__(
        self,
        workers: Optional[Sequence[AsyncContext]] = None,
        *,
        cache_structure: Optional[Sequence[Sequence[CacheBlock]]] = None,
        write_to: Optional[Sequence[CacheBlock]] = None,
    ) -> None:
        if workers is None:
            assert cache_structure is not None, "WorkerGroup needs workers or cache_structure"
            views = [list(v) for v in cache_structure]
            targets = [v[-1] for v in views] if write_to is None else list(write_to)
            assert len(targets) == len(views)
            workers = [AsyncContext(cache_view=v, output_block=t) for v, t in zip(views, targets)]
        else:
            assert cache_structure is None and write_to is None, (
                "pass either workers or cache_structure/write_to, not both"
            )
        self.workers: List[AsyncContext] = list(workers)

        writers = set()
        for ctx in self.workers:
            key = id(ctx.output_block)
            if key in writers:
                raise ValueError("WorkerGroup has two workers writing the same block in one step")
            writers.add(key)

    def __len__(self) -> int:
        return len(self.workers)

    def __iter__(self) -> Iterator[AsyncContext]:
        return iter(self.workers)

    def __getitem__(self, key: Union[int, slice]) -> "AsyncContext | WorkerGroup":
        picked = self.workers[key]
        return WorkerGroup(picked) if isinstance(key, slice) else picked

    @property
    def num_workers(self) -> int:
        return len(self.workers)

    @property
    def cache_structure(self) -> List[List[CacheBlock]]:
        return [list(ctx.cache_view) for ctx in self.workers]

    @property
    def write_to(self) -> List[CacheBlock]:
        return [ctx.output_block for ctx in self.workers]

    def worker_cache_length(self, worker_idx: int) -> int:
        return self.workers[worker_idx].num_cached_tokens

    def max_cache_length(self) -> int:
        return max((ctx.num_cached_tokens for ctx in self.workers), default=0)

    def __repr__(self) -> str:
        distinct = {id(b) for ctx in self.workers for b in ctx.cache_view}
        return f"WorkerGroup(workers={self.num_workers}, blocks={len(distinct)})"
