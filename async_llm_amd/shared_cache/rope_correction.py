"""RoPE rotation of rows by a signed per-row offset, on the GPU.

Same signature and semantics as the reference ``apply_rope_correction``
(``python/minisgl/shared_cache/rope_correction.py:15-54``): neox half-split
pairs, fp32 arithmetic on an fp32 ``cos|sin`` table, ``|offset|`` clamped to
the table, sine negated for negative offsets, one rounding back to the input
dtype.  The work is done by ``va_rope`` in ``libviewattn.so``; tensors must
live on the GPU.
"""

from __future__ import annotations

import torch

from .. import native


def rope_rows(x: torch.Tensor, positions: torch.Tensor, rope: native.VaRope,
              out: torch.Tensor | None = None) -> torch.Tensor:
    """``R(positions) x`` for ``x [N, heads, head_dim]``; ``positions`` is
    int64 ``[N]`` or ``[3, N]`` (3-axis mRoPE)."""
    native.require_device(x, "x")
    assert x.dim() == 3, "expected [rows, heads, head_dim]"
    n, heads, dim = x.shape
    if x.stride(2) != 1 or x.stride(1) != dim:
        x = x.contiguous()
    positions = positions.to(device=x.device, dtype=torch.int64)
    if positions.dim() == 2:
        assert positions.shape == (3, n), f"positions must be [3, {n}]"
        positions = positions.contiguous()
        axis_stride = n
    else:
        assert positions.shape == (n,), f"positions must be [{n}]"
        positions = positions.contiguous()
        axis_stride = 0
    if out is None:
        out = torch.empty((n, heads, dim), dtype=x.dtype, device=x.device)
    native.check(native.lib.va_rope(
        x.data_ptr(), out.data_ptr(), positions.data_ptr(), axis_stride, n, heads, dim,
        native.dtype_id(x.dtype), x.stride(0), out.stride(0), rope,
        native.current_stream_ptr(x.device)))
    return out


def apply_rope_correction(keys: torch.Tensor, corrections: torch.Tensor,
                          cos_sin_cache: torch.Tensor) -> torch.Tensor:
    """Rotate ``keys [N, heads, head_dim]`` by integer offsets ``corrections
    [N]`` (may be negative) using ``cos_sin_cache [max_pos, head_dim]``."""
    native.require_device(keys, "keys")
    cache = cos_sin_cache.to(device=keys.device)
    rope = native.make_rope(keys.shape[-1], cache, None, None)
    out = rope_rows(keys, corrections, rope)
    return out
