"""Paged K/V pool in HBM (reference ``kvcache/mha_pool.py:10-68``).

Layout ``[2, layers, num_pages, page_size, kv_heads, head_dim]``: one token of
one layer is a contiguous ``kv_heads*head_dim`` row, a page is ``page_size``
consecutive rows, so slot ``s`` of layer ``l`` is row ``s`` of the flattened
``[num_pages*page_size, kv_heads*head_dim]`` view the kernels index.
"""

from __future__ import annotations

import torch

from .. import native


class MHAKVCache:
    def __init__(self, num_kv_heads: int, num_layers: int, head_dim: int, num_pages: int,
                 page_size: int, dtype: torch.dtype, device: torch.device) -> None:
        self._kv_buffer = torch.empty(
            (2, num_layers, num_pages, page_size, num_kv_heads, head_dim), device=device, dtype=dtype)
        self._num_layers = num_layers
        self._device = device
        self._rows = num_pages * page_size
        self._width = num_kv_heads * head_dim
        self._shape = native.make_shape(num_kv_heads, num_kv_heads, head_dim, page_size, dtype)

    def k_cache(self, index: int) -> torch.Tensor:
        return self._kv_buffer[0, index]

    def v_cache(self, index: int) -> torch.Tensor:
        return self._kv_buffer[1, index]

    def store_kv(self, k: torch.Tensor, v: torch.Tensor, out_loc: torch.Tensor, layer_id: int) -> None:
        """Scatter rows of ``k``/``v`` to slots ``out_loc`` (negative = skip);
        the HIP counterpart of ``store_cache`` (``kernel/store.py:30-42``)."""
        store_rows(self.k_cache(layer_id), self.v_cache(layer_id), out_loc, k, v)

    @property
    def device(self) -> torch.device:
        return self._device

    @property
    def dtype(self) -> torch.dtype:
        return self._kv_buffer.dtype

    @property
    def num_layers(self) -> int:
        return self._num_layers


def store_rows(k_cache: torch.Tensor, v_cache: torch.Tensor, indices: torch.Tensor,
               k: torch.Tensor, v: torch.Tensor) -> None:
    """``cache[indices[i]] = row i`` for K and V (same argument order as the
    reference ``store_cache``); rows are ``width`` elements, caches may be
    row-strided views."""
    native.require_device(k, "k")
    rows = k_cache.shape[0] if k_cache.dim() == 2 else k_cache.numel() // k.shape[-1]
    width = k.shape[-1]
    k_cache = k_cache.view(rows, -1) if k_cache.is_contiguous() else k_cache
    v_cache = v_cache.view(rows, -1) if v_cache.is_contiguous() else v_cache
    assert k_cache.shape[-1] == width and k_cache.stride(-1) == 1 and v_cache.stride(0) == k_cache.stride(0)
    if k.stride(-1) != 1:
        k = k.contiguous()
    if v.stride(-1) != 1:
        v = v.contiguous()
    n = k.shape[0]
    assert indices.dtype in (torch.int32, torch.int64) and indices.numel() == n
    indices = indices.contiguous()
    shape = native.make_shape(1, 1, width, 1, k.dtype)
    rope = native.VaRope(native.VA_ROPE_TABLE, 0, None, 0, 0, 0, None)
    native.check(native.lib.va_store_kv_rope(
        k.data_ptr(), v.data_ptr(), k.stride(0), v.stride(0), k_cache.data_ptr(), v_cache.data_ptr(),
        k_cache.stride(0), indices.data_ptr(), int(indices.dtype == torch.int64), None, 0,
        n, shape, rope, native.current_stream_ptr(k.device)))
