"""Free list of KV pages (reference ``kvcache/page_allocator.py:6-62``).

Pages are named by the slot of their first token (a multiple of ``page_size``).
"""

from __future__ import annotations

import torch


class PageAllocator:
    def __init__(self, num_pages: int, page_size: int, device: torch.device) -> None:
        self.num_pages = num_pages
        self.page_size = page_size
        self.device = device
        self._free = torch.arange(num_pages, dtype=torch.int32, device=device) * page_size

    @property
    def num_free_pages(self) -> int:
        return int(self._free.numel())

    @property
    def free_page_starts(self) -> torch.Tensor:
        return self._free

    def pages_to_tokens(self, page_starts: torch.Tensor) -> torch.Tensor:
        """``[s, ...] -> [s, s+1, .., s+page_size-1, ...]``."""
        if self.page_size == 1:
            return page_starts
        within = torch.arange(self.page_size, device=page_starts.device, dtype=page_starts.dtype)
        return (page_starts.unsqueeze(1) + within.unsqueeze(0)).reshape(-1)

    def alloc_pages(self, num_pages: int) -> torch.Tensor:
        if num_pages > self.num_free_pages:
            raise RuntimeError(
                f"PageAllocator out of pages: requested {num_pages}, only {self.num_free_pages} free"
            )
        taken, self._free = self._free[:num_pages].clone(), self._free[num_pages:]
        return taken

    def free_pages(self, page_starts: torch.Tensor) -> None:
        if page_starts.numel():
            returned = page_starts.to(device=self._free.device, dtype=self._free.dtype)
            self._free = torch.cat([self._free, returned])
