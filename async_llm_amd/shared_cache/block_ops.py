"""Block merge and append: ``left + right`` as one block whose keys all live in
the left block's position frame.

Mirror of the KV side of the reference session (``python/minisgl/shared_cache/
session.py:330-528``: ``merge_blocks``, ``append_block``, ``_finish_block_merge``,
``_copy_block``, ``_copy_slots``, ``_shift_keys_``) with the same names, argument
meaning and block bookkeeping.  The reference copies K and V layer by layer with
``index_select`` / ``index_copy_`` and then gathers, rotates and scatters the
copied keys once more; here each half of the merge is ONE launch of
``va_copy_shift_kv`` over all layers, which rotates the keys on their way from
the source slots to the destination slots (fp32 rotation, one rounding, as the
reference).

Recurrent (Gated-DeltaNet) block state is not part of the attention path: its
dictionaries are merged with the reference's rules, and composing two affine
summaries is left to the ``compose_affines`` callable of the model that owns
them.
"""

from __future__ import annotations

from typing import Callable, Dict, Optional, Tuple

import numpy as np
import torch

from .. import native
from .shared_block import CacheBlock


def token_slots(block: CacheBlock) -> np.ndarray:
    """Pool slot of every token of ``block`` (host, int64)."""
    if not block.num_tokens:
        return np.empty(0, dtype=np.int64)
    starts = np.asarray(block.page_starts, dtype=np.int64)
    grid = starts[:, None] + np.arange(block.page_size, dtype=np.int64)[None, :]
    return grid.reshape(-1)[: block.num_tokens]


class BlockKVOps:
    """``merge_blocks`` / ``append_block`` over a paged pool.

    ``kv_cache`` offers ``num_layers``, ``k_cache(layer)`` and ``v_cache(layer)``
    (contiguous ``[num_pages, page_size, kv_heads, head_dim]`` tensors on the
    GPU); ``sc_attn`` is the ``SharedCacheAttention`` whose rotation the keys were
    stored with; ``page_allocator`` offers ``alloc_pages(n)``.
    """

    def __init__(self, kv_cache, sc_attn, page_allocator,
                 compose_affines: Optional[Callable[..., Tuple[torch.Tensor, torch.Tensor]]] = None) -> None:
        self.kv_cache = kv_cache
        self.sc_attn = sc_attn
        self.page_allocator = page_allocator
        self.page_size = sc_attn.page_size
        self.device = sc_attn.device
        self.compose_affines = compose_affines
        self._refs: tuple = ()

    def create_block(self) -> CacheBlock:
        return CacheBlock(self.device, self.page_size)

    # ------------------------------------------------------------------
    def merge_blocks(self, left: CacheBlock, right: CacheBlock) -> CacheBlock:
        """Copy ``left + right`` into a new compact block; both inputs stay
        valid and unchanged (reference ``session.py:330-377``)."""
        self._validate_block(left)
        self._validate_block(right)
        left_tokens, right_tokens = left.num_tokens, right.num_tokens
        left_span, right_span = left.mrope_span, right.mrope_span
        total_tokens = left_tokens + right_tokens

        merged = self.create_block()
        num_pages = -(-total_tokens // self.page_size)
        if num_pages:
            merged.page_starts = self.page_allocator.alloc_pages(num_pages).tolist()
        merged.num_tokens = total_tokens

        if left_tokens:
            self._copy_block(left, merged, destination_start=0)
        if right_tokens:
            self._copy_slots(token_slots(right), merged, destination_start=left_tokens, position_shift=left_span)
        self._finish_block_merge(destination=merged, left=left, right=right, left_span=left_span,
                                 right_span=right_span, keep_left_state=False)
        return merged

    def append_block(self, left: CacheBlock, right: CacheBlock) -> CacheBlock:
        """Append a copy of ``right`` to ``left`` and return ``left``; the free
        slots of ``left``'s last page are filled first.  ``append_block(b, b)``
        doubles ``b`` in place (reference ``session.py:379-420``)."""
        self._validate_block(left)
        self._validate_block(right)
        left_tokens, right_tokens = left.num_tokens, right.num_tokens
        left_span, right_span = left.mrope_span, right.mrope_span
        if right_tokens:
            # the source layout is taken before ``left`` grows: they may be the same object
            source_slots = token_slots(right)
            new_pages = self.page_allocator.alloc_pages(left.pages_needed(right_tokens))
            left.grow_pages(new_pages, right_tokens)
            self._copy_slots(source_slots, left, destination_start=left_tokens, position_shift=left_span)
        self._finish_block_merge(destination=left, left=left, right=right, left_span=left_span,
                                 right_span=right_span, keep_left_state=True)
        return left

    # ------------------------------------------------------------------
    def _finish_block_merge(self, *, destination: CacheBlock, left: CacheBlock, right: CacheBlock, left_span: int,
                            right_span: int, keep_left_state: bool) -> None:
        """Token ids, span and recurrent state of the result (reference
        ``session.py:422-477``)."""
        destination.token_ids = [*list(left.token_ids), *right.token_ids]
        merged_span = left_span + right_span
        destination.mrope_span_override = None if merged_span == destination.num_tokens else merged_span

        merged_affine: Dict[int, Tuple[torch.Tensor, torch.Tensor]] = {}
        for layer_idx in set(left.linear_affine) | set(right.linear_affine):
            left_pair = left.linear_affine.get(layer_idx)
            right_pair = right.linear_affine.get(layer_idx)
            if left_pair is None:
                merged_affine[layer_idx] = (right_pair[0].clone(), right_pair[1].clone())
            elif right_pair is None:
                merged_affine[layer_idx] = left_pair if keep_left_state else (left_pair[0].clone(), left_pair[1].clone())
            else:
                if self.compose_affines is None:
                    raise NotImplementedError(
                        "both blocks carry recurrent state for layer %d: pass compose_affines "
                        "(the model's composition of two affine summaries)" % layer_idx)
                merged_affine[layer_idx] = self.compose_affines(A_first=left_pair[0], B_first=left_pair[1],
                                                                A_second=right_pair[0], B_second=right_pair[1])
        merged_conv: Dict[int, torch.Tensor] = {}
        for layer_idx in set(left.linear_conv_state) | set(right.linear_conv_state):
            right_state = right.linear_conv_state.get(layer_idx)
            state = right_state if right_state is not None else left.linear_conv_state.get(layer_idx)
            merged_conv[layer_idx] = state if keep_left_state and right_state is None else state.clone()
        destination._replace_linear_states(merged_affine, merged_conv)

    def _validate_block(self, block: CacheBlock) -> None:
        if block.device != self.device:
            raise ValueError("block must belong to this session's device")
        if block.page_size != self.page_size:
            raise ValueError("block must use this session's page size")

    def _copy_block(self, source: CacheBlock, destination: CacheBlock, destination_start: int) -> None:
        """Copy all KV of ``source`` into one range of ``destination``."""
        self._copy_slots(token_slots(source), destination, destination_start)

    def _copy_slots(self, source_slots, destination: CacheBlock, destination_start: int,
                    position_shift: int = 0) -> None:
        """Copy KV from the given pool slots into ``destination`` from token
        ``destination_start`` on, in every layer; with ``position_shift`` the
        copied keys are rotated by it on the way (the reference's
        ``_copy_slots`` followed by ``_shift_keys_``)."""
        source = np.asarray(torch.as_tensor(source_slots).cpu(), dtype=np.int64).reshape(-1)
        n = source.size
        if n == 0:
            return
        target = token_slots(destination)[destination_start: destination_start + n]
        assert target.size == n, "destination block is too short for the copied run"
        # the kernel scatters while it gathers: a slot read by one token and written by another would race
        if np.intersect1d(source, target).size:
            raise ValueError("source and destination slots of a block copy overlap")
        self._launch(source, target, int(position_shift))

    def _shift_keys_(self, *, block: CacheBlock, start: int, num_tokens: int, position_shift: int) -> None:
        """Rotate stored keys ``[start, start + num_tokens)`` of ``block`` by
        ``position_shift`` in place (reference ``session.py:509-528``).  Merge and
        append do not need it here (the copy rotates); kept for callers that
        re-frame a block without copying it."""
        slots = token_slots(block)[start: start + num_tokens]
        if slots.size and position_shift:
            # source == destination row by row: every thread rewrites the pieces it read (the value
            # rows are rewritten unchanged)
            self._launch(slots, slots, int(position_shift))

    # ------------------------------------------------------------------
    def _launch(self, source: np.ndarray, target: np.ndarray, position_shift: int) -> None:
        att = self.sc_attn
        n = source.size
        host = torch.from_numpy(np.stack([source, target]))
        if self.device.type != "cuda":
            raise native.ViewAttnError("block copies run on the GPU only (HIP kernel, no CPU path)")
        host = host.pin_memory()
        dev = host.to(self.device, non_blocking=True)
        self._refs = (host, dev)  # alive until the next copy on this stream has been queued
        L = self.kv_cache.num_layers
        k0, v0 = self.kv_cache.k_cache(0), self.kv_cache.v_cache(0)
        assert k0.is_contiguous() and v0.is_contiguous(), "pool layers must be contiguous"
        width = att.num_kv_heads * att.head_dim
        item = k0.element_size()
        groups = [(0, L, 0)]
        if L > 1:
            k_step = self.kv_cache.k_cache(1).data_ptr() - k0.data_ptr()
            v_step = self.kv_cache.v_cache(1).data_ptr() - v0.data_ptr()
            uniform = k_step == v_step and k_step % item == 0 and all(
                self.kv_cache.k_cache(l).data_ptr() == k0.data_ptr() + l * k_step
                and self.kv_cache.v_cache(l).data_ptr() == v0.data_ptr() + l * k_step for l in range(2, L))
            groups = [(0, L, k_step // item)] if uniform else [(l, 1, 0) for l in range(L)]
        rope = att._rope_descriptor() if position_shift else None
        stream = native.current_stream_ptr(self.device)
        for first, count, stride in groups:
            k_pool, v_pool = self.kv_cache.k_cache(first), self.kv_cache.v_cache(first)
            native.check(native.lib.va_copy_shift_kv(
                k_pool.data_ptr(), v_pool.data_ptr(), width, stride, count, dev[0].data_ptr(), dev[1].data_ptr(),
                n, position_shift, att._shape, rope, stream))
