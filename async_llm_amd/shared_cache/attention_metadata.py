"""Host-side page tables for one ``prepare`` call.

Parity with the reference ``page_numbers`` / ``upload_page_indices``
(``python/minisgl/shared_cache/attention_metadata.py:12-40``): tables are
bit-exact; each distinct block's page list is walked once per prepare.
"""

from __future__ import annotations

from typing import Dict, List, Optional

import numpy as np
import torch


def page_numbers(block, snapshot: Dict[int, List[int]], extra_page: Optional[int] = None) -> List[int]:
    """Page numbers (``page_start // page_size``) of ``block``, plus the page
    this step's token is about to open (``extra_page``, a page-start slot).

    ``snapshot`` belongs to the calling prepare: the first request for a block
    fixes its list (pending page included), later requests return that same
    list object.  The block itself is never modified.
    """
    key = id(block)
    cached = snapshot.get(key)
    if cached is None:
        size = block.page_size
        cached = [start // size for start in block.page_starts]
        if extra_page is not None:
            cached.append(extra_page // size)
        snapshot[key] = cached
    return cached


def page_array(block) -> np.ndarray:
    """int32 page numbers of ``block`` as an array, kept on the block between
    prepares: converting a Python page list costs more per element than every
    other step of planning.  Blocks that count their page-list changes
    (``_pages_version``) are served from the cache while version, length and last
    entry are unchanged, and a list that only grew is extended by its new tail;
    any other block object is converted afresh."""
    starts = block.page_starts
    n = len(starts)
    version = getattr(block, "_pages_version", None)
    if version is None:
        return (np.asarray(starts, dtype=np.int64) // block.page_size).astype(np.int32)
    key = (version, n, starts[-1] if n else None)
    cached = getattr(block, "_page_array_cache", None)
    if cached is not None and cached[0] == key:
        return cached[1]
    arr = (np.asarray(starts, dtype=np.int64) // block.page_size).astype(np.int32)
    arr.setflags(write=False)
    block._page_array_cache = (key, arr)
    return arr


def page_numbers_array(block, snapshot: Dict[int, np.ndarray], extra_page: Optional[int] = None) -> np.ndarray:
    """``page_numbers`` as an int32 array (same values, same snapshot rule)."""
    key = id(block)
    cached = snapshot.get(key)
    if cached is None:
        cached = page_array(block)
        if extra_page is not None:
            cached = np.append(cached, np.int32(extra_page // block.page_size))
        snapshot[key] = cached
    return cached


def upload_page_indices(parts, device: torch.device, refs: List[torch.Tensor]) -> torch.Tensor:
    """Concatenate per-segment page lists (lists or int arrays) into one int32
    table on ``device``.

    The host staging tensor is pinned when the target is a GPU and the copy is
    asynchronous, so both tensors are appended to ``refs`` (host first, device
    second): the caller keeps them alive until the stream has consumed them.
    """
    total = sum(len(part) for part in parts)
    host = torch.empty(total, dtype=torch.int32, device="cpu", pin_memory=device.type == "cuda")
    if total:
        np.concatenate([np.asarray(part, dtype=np.int32) for part in parts], out=host.numpy())
    table = host.to(device, non_blocking=True)
    refs.append(host)
    refs.append(table)
    return table
