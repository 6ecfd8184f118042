"""GPU: rotation and KV store against the oracle.  Cases follow the reference's
tests/core/test_rope_correction_kernel.py, test_shared_cache.py:178-258 and
tests/kernel/test_store_padding.py."""

import pytest
import torch

from async_llm_amd import native
from async_llm_amd.kvcache.mha_pool import store_rows
from async_llm_amd.shared_cache import apply_rope_correction
from async_llm_amd.shared_cache.rope_correction import rope_rows
from oracle import view_attention_oracle as O

pytestmark = pytest.mark.gpu
DEV = "cuda"


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("heads,dim", [(4, 64), (2, 128), (3, 256)])
def test_rope_correction_matches_oracle_bit_exact(dtype, heads, dim):
    torch.manual_seed(0)
    keys = torch.randn(8, heads, dim).to(dtype)
    corr = torch.tensor([0, 5, -3, 17, -12, 42, 255, -300])  # last two reach / pass the table end
    cs = O.build_cos_sin_cache(dim, 256, 10000.0)
    got = apply_rope_correction(keys.to(DEV), corr.to(DEV), cs.to(DEV))
    want = O.apply_rope_correction(keys, corr, cs)
    assert got.dtype == dtype and got.shape == keys.shape
    assert torch.equal(got.cpu(), want)


def test_rope_identity_roundtrip_empty_and_in_place():
    torch.manual_seed(1)
    cs = O.build_cos_sin_cache(64, 128, 10000.0).to(DEV)
    keys = torch.randn(5, 2, 64, device=DEV)
    assert torch.equal(apply_rope_correction(keys, torch.zeros(5, dtype=torch.int64, device=DEV), cs), keys)
    fwd = apply_rope_correction(keys, torch.full((5,), 23, device=DEV), cs)
    back = apply_rope_correction(fwd, torch.full((5,), -23, device=DEV), cs)
    assert torch.allclose(back, keys, atol=1e-5)
    empty = apply_rope_correction(torch.zeros(0, 2, 64, device=DEV), torch.zeros(0, dtype=torch.int64, device=DEV), cs)
    assert empty.shape == (0, 2, 64)
    rope = native.make_rope(64, cs, None, None)
    work = keys.clone()
    rope_rows(work, torch.full((5,), 23, device=DEV), rope, out=work)
    assert torch.equal(work, fwd)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_partial_rotary_and_mrope_match_oracle(dtype):
    torch.manual_seed(2)
    x = torch.randn(9, 4, 128).to(dtype)
    pos = torch.tensor([0, 1, 7, 30, 4, 100, 12352, 70000, 3])
    cs = O.build_cos_sin_cache(32, 128, 1e6)
    cs_dev = cs.to(DEV)
    got = rope_rows(x.to(DEV), pos.to(DEV), native.make_rope(32, cs_dev, None, None))
    assert torch.equal(got.cpu(), O.rope_partial(x, pos, cs, 32))
    inv = O.mrope_inv_freq(64, 1e7)
    rope = native.make_rope(64, None, inv.to(DEV), (12, 10, 10))
    atol = 1e-5 if dtype == torch.float32 else 2e-2
    for p in (pos, torch.stack([pos, pos * 2 + 1, pos + 3])):
        got = rope_rows(x.to(DEV), p.to(DEV), rope)
        want = O.rope_mrope(x, p, inv, (12, 10, 10), 64)
        # cos/sin come from the device's own sincos: values agree to rounding, not bit for bit
        assert torch.allclose(got.cpu().float(), want.float(), atol=atol, rtol=1e-2 if dtype != torch.float32 else 1e-5)
        assert torch.equal(got.cpu()[..., 64:], x[..., 64:])


@pytest.mark.parametrize("index_dtype", [torch.int32, torch.int64])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
def test_store_skips_negative_slots_and_touches_nothing_else(index_dtype, dtype):
    backing = torch.full((12, 2, 128), 7, device=DEV, dtype=dtype)
    cache = backing[2:-1]
    for slots in ([0, -1, 3, -2], [-1, 8, -1, 2], [-1, -1, -1, -1], [1, 2, 3, 4]):
        backing.fill_(7)
        qkv = torch.randn(4, 4 * 128, device=DEV).to(dtype)
        key, value = qkv[:, :128], qkv[:, 128:256]  # row-strided views of a fused projection
        idx = torch.tensor(slots, device=DEV, dtype=index_dtype)
        store_rows(cache[:, 0], cache[:, 1], idx, key, value)
        expected = torch.full_like(backing, 7)
        for row, slot in enumerate(slots):
            if slot >= 0:
                expected[slot + 2, 0] = key[row]
                expected[slot + 2, 1] = value[row]
        assert torch.equal(backing, expected)
