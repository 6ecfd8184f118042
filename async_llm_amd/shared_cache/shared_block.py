"""Paged cache blocks: the unit a cache view is assembled from.

Interface parity with the reference ``CacheBlock``
(``python/minisgl/shared_cache/shared_block.py:24-195``): same attribute and
method names, same page arithmetic, same assertion messages where the
reference's tests match on them.  Pure host-side bookkeeping; no device work.

Storage rule: block-relative token ``i`` sits in pool slot
``page_starts[i // page_size] + i % page_size``; only the final page may be
partly filled.  Keys are stored rotated to block-relative positions and are
never rewritten when the block is viewed from a different place in a view.
"""

from __future__ import annotations

import itertools
from typing import Dict, Iterable, List, Optional, Tuple

import torch


class StateCache:
    """Holder of a lazily prepared Gated-DeltaNet address table (reference
    ``gdn_state.py:9-11``).  The attention path never reads it; it exists so
    reference GDN code handed one of these blocks keeps working."""

    def __init__(self) -> None:
        self.prepared = None


class StateDict(dict):
    """``dict`` that drops the owner's prepared state on every mutation
    (reference ``gdn_state.py:14-58``)."""

    def __init__(self, cache: StateCache, values: Iterable = ()) -> None:
        super().__init__(values)
        self.cache = cache

    def _touch(self) -> None:
        self.cache.prepared = None

    def __setitem__(self, key, value) -> None:
        self._touch()
        super().__setitem__(key, value)

    def __delitem__(self, key) -> None:
        self._touch()
        super().__delitem__(key)

    def clear(self) -> None:
        self._touch()
        super().clear()

    def pop(self, key, *default):
        self._touch()
        return super().pop(key, *default)

    def popitem(self):
        self._touch()
        return super().popitem()

    def update(self, *args, **kwargs) -> None:
        self._touch()
        super().update(*args, **kwargs)

    def setdefault(self, key, default=None):
        if key not in self:
            self._touch()
        return super().setdefault(key, default)

    def __ior__(self, other):
        self.update(other)
        return self


_block_ids = itertools.count()


class CacheBlock:
    """A growable run of KV tokens backed by pages borrowed from the pool.

    ``page_starts`` holds the slot of the first token of every owned page (a
    multiple of ``page_size``); ``num_tokens`` counts the valid tokens;
    ``token_ids`` mirrors the stored tokens on the host.  ``mrope_span`` is how
    far the running (m)RoPE position advances across the block: the token
    count for text, or ``mrope_span_override`` when an image compressed it.
    """

    def __init__(self, device: torch.device, page_size: int = 1) -> None:
        self.block_id = next(_block_ids)
        self.device = device
        self.page_size = page_size
        self._pages_version = 0  # bumped by every change of the page list: keys the planners' page-table cache
        self.page_starts = []
        self.num_tokens: int = 0
        self.token_ids: List[int] = []
        self.mrope_span_override: Optional[int] = None
        # Gated-DeltaNet pass-through state (unused by view attention).
        self._gdn_state_cache = StateCache()
        self.linear_affine = StateDict(self._gdn_state_cache)
        self.linear_conv_state = StateDict(self._gdn_state_cache)

    # -- GDN pass-through -------------------------------------------------
    def invalidate_gdn_state(self) -> None:
        self._gdn_state_cache.prepared = None

    @property
    def linear_affine(self) -> Dict[int, Tuple[torch.Tensor, torch.Tensor]]:
        return self._linear_affine

    @linear_affine.setter
    def linear_affine(self, value) -> None:
        self.invalidate_gdn_state()
        self._linear_affine = value

    @property
    def linear_conv_state(self) -> Dict[int, torch.Tensor]:
        return self._linear_conv_state

    @linear_conv_state.setter
    def linear_conv_state(self, value) -> None:
        self.invalidate_gdn_state()
        self._linear_conv_state = value

    def _replace_linear_states(self, affine, conv) -> None:
        self.linear_affine = StateDict(self._gdn_state_cache, affine)
        self.linear_conv_state = StateDict(self._gdn_state_cache, conv)

    # -- page list --------------------------------------------------------
    @property
    def page_starts(self) -> List[int]:
        return self._page_starts

    @page_starts.setter
    def page_starts(self, value: List[int]) -> None:
        self._page_starts = value
        self._pages_version += 1

    # -- page arithmetic --------------------------------------------------
    @property
    def mrope_span(self) -> int:
        override = self.mrope_span_override
        return self.num_tokens if override is None else override

    @property
    def num_pages(self) -> int:
        return len(self.page_starts)

    @property
    def last_page_len(self) -> int:
        """Tokens in the final page: ``1..page_size``, or 0 for an empty block."""
        if not self.num_tokens:
            return 0
        return self.num_tokens - self.page_size * (self.num_pages - 1)

    @property
    def free_tail(self) -> int:
        """Unused slots at the end of the final page."""
        return self.page_size * self.num_pages - self.num_tokens

    @property
    def has_capacity(self) -> bool:
        return self.free_tail > 0

    def pages_needed(self, num_new_tokens: int) -> int:
        """Fresh pages required to append ``num_new_tokens`` (the free tail of
        the final page is consumed first)."""
        overflow = num_new_tokens - self.free_tail
        return 0 if overflow <= 0 else -(-overflow // self.page_size)

    # -- device views of the tables (not used by the planners) ------------
    def page_starts_tensor(self) -> torch.Tensor:
        return torch.tensor(self.page_starts, dtype=torch.int32, device=self.device)

    def page_numbers_tensor(self) -> torch.Tensor:
        return self.page_starts_tensor() // self.page_size

    def token_slots_tensor(self) -> torch.Tensor:
        if not self.num_tokens:
            return torch.empty(0, dtype=torch.int32, device=self.device)
        within = torch.arange(self.page_size, dtype=torch.int32, device=self.device)
        grid = self.page_starts_tensor().unsqueeze(1) + within.unsqueeze(0)
        return grid.reshape(-1)[: self.num_tokens]

    # -- growth -----------------------------------------------------------
    def grow_pages(self, page_starts: torch.Tensor, num_new_tokens: int) -> None:
        """Commit a prefill write of ``num_new_tokens`` tokens that took
        ``page_starts`` fresh pages after filling the free tail."""
        assert num_new_tokens > 0, "grow_pages needs at least one token"
        expected = self.pages_needed(num_new_tokens)
        assert page_starts.numel() == expected, (
            f"grow_pages got {page_starts.numel()} pages for {num_new_tokens} tokens "
            f"(free tail {self.free_tail}, page_size {self.page_size}); expected {expected}"
        )
        self.page_starts += [int(s) for s in page_starts.tolist()]
        self.num_tokens += num_new_tokens

    def append_token(self, new_page_start: Optional[int]) -> None:
        """Commit one decode write; ``new_page_start`` is given exactly when
        the token opens a new page."""
        if new_page_start is None:
            assert self.has_capacity, "append_token needs a new page but none was given"
        else:
            assert not self.has_capacity, "append_token got a new page but last page has room"
            self.page_starts.append(int(new_page_start))
            self._pages_version += 1
        self.num_tokens += 1
        if self.mrope_span_override is not None:
            # decoded tokens are text: the frame advances by one with them
            self.mrope_span_override += 1

    def clear(self) -> List[int]:
        """Empty the block; returns the page-start slots to hand back."""
        self.invalidate_gdn_state()
        released = list(self.page_starts)
        self.page_starts.clear()
        self._pages_version += 1
        self.token_ids.clear()
        self.num_tokens = 0
        self.mrope_span_override = None
        self.linear_affine.clear()
        self.linear_conv_state.clear()
        return released

    def __repr__(self) -> str:
        return (
            f"CacheBlock(id={self.block_id}, tokens={self.num_tokens}, "
            f"pages={self.num_pages}, page_size={self.page_size})"
        )


SharedBlock = CacheBlock
