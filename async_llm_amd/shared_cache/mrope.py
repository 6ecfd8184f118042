"""Interleaved-mRoPE positions of a flat token sequence (host side).

Same result as the reference ``get_rope_index``
(``python/minisgl/models/qwen3_5_mrope.py:19-64``): a text run advances all
three axes together; an image of grid ``(t, h, w)`` places its ``t*(h/m)*(w/m)``
tokens on a (temporal, height, width) lattice starting at the running position
and advances that position by ``max(h, w) // m`` only.
"""

from __future__ import annotations

from typing import Optional

import torch


def _image_lattice(start: int, t: int, h: int, w: int, merge: int, device) -> torch.Tensor:
    rows, cols = h // merge, w // merge
    frame = torch.arange(t, device=device).repeat_interleave(rows * cols)
    row = torch.arange(rows, device=device).repeat_interleave(cols).repeat(t)
    col = torch.arange(cols, device=device).repeat(rows * t)
    return torch.stack([frame, row, col]) + start


def get_rope_index(
    input_ids: torch.Tensor,
    mm_token_type_ids: torch.Tensor,
    spatial_merge_size: int,
    image_grid_thw: Optional[torch.Tensor] = None,
) -> torch.Tensor:
    """``[3, T]`` positions for ``input_ids [T]``; ``mm_token_type_ids`` marks
    text (0), image (1) or video (2) tokens."""
    device = input_ids.device
    kinds = mm_token_type_ids.tolist()
    grids = [] if image_grid_thw is None else image_grid_thw.tolist()
    pieces, cursor, next_grid, i = [], 0, 0, 0
    while i < len(kinds):
        j = i
        while j < len(kinds) and kinds[j] == kinds[i]:
            j += 1
        if kinds[i] == 0:
            pieces.append(torch.arange(cursor, cursor + (j - i), device=device).unsqueeze(0).expand(3, -1))
            cursor += j - i
        elif kinds[i] in (1, 2):
            t, h, w = (int(x) for x in grids[next_grid])
            next_grid += 1
            pieces.append(_image_lattice(cursor, t, h, w, spatial_merge_size, device))
            cursor += max(h, w) // spatial_merge_size
        else:
            raise NotImplementedError(f"Unexpected mm_token_type_ids entry == {kinds[i]}")
        i = j
    return torch.cat(pieces, dim=1).reshape(3, -1)
