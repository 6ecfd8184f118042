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


def test_new_rows_can_go_through_the_pools_own_store_kv():
    """``fused_store=False``: the op rotates the new keys and hands K and V to ``kv_cache.store_kv`` as the
    reference does (``attention.py:645-649``) instead of writing the pool itself -- for pools whose
    ``store_kv`` does more than copy rows.  Same pool contents, same attention result, and the pool's method
    is what ran."""
    from types import SimpleNamespace

    from async_llm_amd import workloads
    from async_llm_amd.shared_cache import SharedCacheAttention

    dev = torch.device("cuda")
    wl = workloads.batched_decode(dev, workers=5, shared_len=300, private_lo=20, private_hi=200, heads=(8, 2, 64))
    op = wl.op
    want = op.forward(wl.q, wl.k, wl.v, 0, wl.batch)
    want_k = wl.pool.k_cache(0).clone()
    want_v = wl.pool.v_cache(0).clone()
    # a second pool, same contents before the step, whose store_kv counts its calls
    calls = []
    k2, v2 = wl.pool.k_cache(0).clone(), wl.pool.v_cache(0).clone()
    slots = wl.new_token_slots.long()
    k2.view(-1, k2.shape[-2] * k2.shape[-1])[slots] = 0
    v2.view(-1, v2.shape[-2] * v2.shape[-1])[slots] = 0

    def store_kv(k, v, out_loc, layer_id):
        calls.append(layer_id)
        k2.view(-1, k.shape[-1])[out_loc.long()] = k
        v2.view(-1, v.shape[-1])[out_loc.long()] = v

    pool = SimpleNamespace(k_cache=lambda layer: k2, v_cache=lambda layer: v2, store_kv=store_kv)
    other = SharedCacheAttention(pool, op.cos_sin_cache, op.num_qo_heads, op.num_kv_heads, op.head_dim, op.page_size,
                                 op.dtype, dev, rotary_dim=op.rotary_dim, fused_store=False)
    meta = other.prepare(wl.group, wl.pending, wl.new_token_slots)
    batch = SimpleNamespace(attn_metadata=meta, positions=wl.batch.positions, out_loc=wl.batch.out_loc, mrope_positions=None)
    got = other.forward(wl.q, wl.k, wl.v, 0, batch)
    torch.cuda.synchronize()
    assert calls == [0]
    assert torch.equal(k2, want_k) and torch.equal(v2, want_v)
    assert torch.equal(got, want)
