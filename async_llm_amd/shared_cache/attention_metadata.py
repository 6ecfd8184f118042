"""Host-side page tables for one ``prepare`` call.

Parity with the reference ``page_numbers`` / ``upload_page_indices``
(``python/minisgl/shared_cache/attention_metadata.py:12-40``): tables are
bit-exact; each distinct block's page list is walked once per prepare.
"""

from __future__ import annotations

from typing import Dict, List, Optional

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


def upload_page_indices(parts, device: torch.device, refs: List[torch.Tensor]) -> torch.Tensor:
    """Concatenate per-segment page lists into one int32 table on ``device``.

    The host staging tensor is pinned when the target is a GPU and the copy is
    asynchronous, so both tensors are appended to ``refs`` (host first, device
    second): the caller keeps them alive until the stream has consumed them.
    """
    flat = [page for part in parts for page in part]
    host = torch.tensor(flat, dtype=torch.int32, device="cpu", pin_memory=device.type == "cuda")
    table = host.to(device, non_blocking=True)
    refs.append(host)
    refs.append(table)
    return table
