"""Slot and page planning a caller performs around the attention op.

These mirror the helpers of the reference session
(``python/minisgl/shared_cache/session.py:1078-1141``) so a harness can drive
``SharedCacheAttention`` exactly as the session does.
"""

from __future__ import annotations

from typing import Dict, List, Optional, Tuple

import torch


def plan_decode_writes(group, page_size: int, page_allocator, device) -> Tuple[Dict[int, Optional[int]], torch.Tensor, List[int]]:
    """For one decode step pick each worker's destination slot.

    Returns ``(new_page_for_block, new_token_slots, write_pos)``:
    ``id(block) -> page-start slot`` of a freshly borrowed page (``None`` when
    the token fits the last page), the int32 slot of every new token, and the
    block-relative write position (the block's mRoPE span).  All blocks that
    need a page share ONE allocator call and one host read-back.
    """
    targets = group.write_to
    pending: Dict[int, Optional[int]] = {}
    starved = []
    for block in targets:
        if id(block) in pending:
            raise ValueError("WorkerGroup has two workers writing the same block in one step")
        pending[id(block)] = None
        if not block.has_capacity:
            starved.append(block)
    if starved:
        fresh = page_allocator.alloc_pages(len(starved)).cpu().tolist()
        for block, start in zip(starved, fresh):
            pending[id(block)] = start
    slots, positions = [], []
    for block in targets:
        opened = pending[id(block)]
        base = block.page_starts[-1] if opened is None else opened
        slots.append(base + block.num_tokens % page_size)
        positions.append(block.mrope_span)
    return pending, torch.tensor(slots, dtype=torch.int32, device=device), positions


def alloc_token_storage(seq_len: int, page_size: int, page_allocator, device,
                        write_to=None) -> Tuple[torch.Tensor, torch.Tensor]:
    """Borrow the pages for ``seq_len`` new tokens of ``write_to`` and return
    ``(new_page_starts, token_slots)``; the free tail of the block's last page
    is used before any new page."""
    tail = 0 if write_to is None else write_to.free_tail
    fresh = page_allocator.alloc_pages(-(-max(0, seq_len - tail) // page_size))
    new_slots = page_allocator.pages_to_tokens(fresh)
    if tail == 0:
        return fresh, new_slots[:seq_len]
    first = write_to.page_starts[-1] + write_to.last_page_len
    tail_slots = torch.arange(first, first + tail, dtype=new_slots.dtype, device=device)
    return fresh, torch.cat([tail_slots, new_slots])[:seq_len]
