"""The oracle's block merge / append (the checker of ``va_copy_shift_kv``) pinned
by what the operation must mean: a merged block read as ONE segment gives the
same attention as the closed-form softmax over ``left + right`` at absolute
positions (the reference's own criterion, tests/core/test_cache_block_merge.py:
146-171 "merged block matches split view"), append equals merge slot for slot
and self-append doubles the block (same file :174-226), a zero shift is a plain
copy.  Host bookkeeping of the product's ``BlockKVOps`` is checked without a GPU
up to the launch."""

import pytest
import torch

from async_llm_amd import native
from async_llm_amd.shared_cache import BlockKVOps, CacheBlock
from async_llm_amd.shared_cache.block_ops import token_slots
from oracle import view_attention_oracle as O

BASE = 10000.0


class Alloc:
    def __init__(self, page, first):
        self.page, self.next = page, first

    def __call__(self, n):
        got = [(self.next + i) * self.page for i in range(n)]
        self.next += n
        return got

    def alloc_pages(self, n):
        return torch.tensor(self(n), dtype=torch.int32)


def filled_block(alloc, page, n, span=None):
    b = O.OBlock(page)
    if n:
        b.grow_pages(alloc(b.pages_needed(n)), n)
    b.mrope_span_override = span
    return b


def store_raw(pools, block, raw_k, raw_v, rel_pos, rope):
    slots = torch.tensor(block.token_slots())
    k_pool, v_pool = pools
    k_pool[slots] = rope.rotate(raw_k, rel_pos).to(k_pool.dtype)
    v_pool[slots] = raw_v.to(v_pool.dtype)


@pytest.mark.parametrize("rotary", [16, 8])
@pytest.mark.parametrize("left_span,right_span", [(None, None), (4, 3)])
@pytest.mark.parametrize("append", [False, True])
def test_merged_block_read_as_one_segment_matches_the_closed_form(rotary, left_span, right_span, append):
    page, Hq, Hkv, D, nl, nr = 4, 4, 2, 16, 7, 5
    g = torch.Generator().manual_seed(5)
    rope = O.RopeSpec(rotary, O.build_cos_sin_cache(rotary, 64, BASE))
    k_pool = torch.zeros(64 * page, Hkv, D)
    v_pool = torch.zeros(64 * page, Hkv, D)
    alloc = Alloc(page, 1)
    left, right = filled_block(alloc, page, nl, left_span), filled_block(alloc, page, nr, right_span)
    raw = {name: torch.randn(n, Hkv, D, generator=g) for name, n in (("lk", nl), ("lv", nl), ("rk", nr), ("rv", nr))}
    # compressed spans: several tokens share a position, as the patches of an image do
    rel_l = torch.arange(nl) if left_span is None else torch.tensor([0, 1, 1, 1, 2, 2, 3])
    rel_r = torch.arange(nr) if right_span is None else torch.tensor([0, 0, 1, 2, 2])
    store_raw((k_pool, v_pool), left, raw["lk"], raw["lv"], rel_l, rope)
    store_raw((k_pool, v_pool), right, raw["rk"], raw["rv"], rel_r, rope)
    span_l, span_r = left.mrope_span, right.mrope_span
    if append:
        merged = O.append_block([(k_pool, v_pool)], left, right, alloc, rope)
        assert merged is left
    else:
        merged = O.merge_blocks([(k_pool, v_pool)], left, right, alloc, rope)
    assert merged.num_tokens == nl + nr and merged.mrope_span == span_l + span_r

    own = O.OBlock(page)
    pending, slots, write_pos = O.plan_decode_writes([own], page, alloc)
    plan = O.plan_decode([[merged, own]], [own], pending, slots, page)
    q = torch.randn(1, Hq, D, generator=g)
    new_k, new_v = torch.randn(1, Hkv, D, generator=g), torch.randn(1, Hkv, D, generator=g)
    O.store_kv(k_pool.view(-1, Hkv * D), v_pool.view(-1, Hkv * D), torch.tensor(slots),
               rope.rotate(new_k, torch.tensor(write_pos)).reshape(1, -1), new_v.reshape(1, -1))
    out, lse, _ = O.forward_decode(plan, q, k_pool.view(-1, page, Hkv, D), v_pool.view(-1, page, Hkv, D), rope)
    total = span_l + span_r
    exp_out, exp_lse = O.concat_view_attention(
        q[0], total, [raw["lk"], raw["rk"], new_k], [raw["lv"], raw["rv"], new_v], [0, span_l, total],
        [rel_l, rel_r, torch.zeros(1, dtype=torch.int64)], rotary, BASE)
    torch.testing.assert_close(out.view(Hq, D).double(), exp_out, atol=2e-5, rtol=2e-5)
    torch.testing.assert_close(lse.view(Hq).double(), exp_lse, atol=2e-5, rtol=2e-5)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("mrope", [False, True])
def test_append_equals_merge_and_self_append_doubles(dtype, mrope):
    page, Hkv, D, rotary = 4, 2, 16, 8
    g = torch.Generator().manual_seed(6)
    rope = (O.RopeSpec(rotary, None, (2, 1, 1), O.mrope_inv_freq(rotary, BASE)) if mrope
            else O.RopeSpec(rotary, O.build_cos_sin_cache(rotary, 64, BASE)))
    layers = [(torch.randn(48 * page, Hkv, D, generator=g).to(dtype), torch.randn(48 * page, Hkv, D, generator=g).to(dtype))
              for _ in range(2)]
    alloc = Alloc(page, 1)
    left, right = filled_block(alloc, page, 6, 5), filled_block(alloc, page, 9)
    before = [(k.clone(), v.clone()) for k, v in layers]
    merged = O.merge_blocks(layers, left, right, alloc, rope)
    for (k, v), (k0, v0) in zip(layers, before):  # the inputs are untouched
        for b in (left, right):
            s = torch.tensor(b.token_slots())
            assert torch.equal(k[s], k0[s]) and torch.equal(v[s], v0[s])
    left_pages = list(left.page_starts)
    appended = O.append_block(layers, left, right, alloc, rope)
    assert appended is left and left.page_starts[: len(left_pages)] == left_pages
    assert left.num_tokens == 15 and left.mrope_span == 14 and merged.mrope_span == 14
    ms, ls = torch.tensor(merged.token_slots()), torch.tensor(left.token_slots())
    for k, v in layers:
        assert torch.equal(k[ms], k[ls]) and torch.equal(v[ms], v[ls])
    # the right half is the right block's keys rotated by the left span, values copied
    rs = torch.tensor(right.token_slots())
    for k, v in layers:
        assert torch.equal(v[ms[6:]], v[rs])
        expect = rope.rotate(k[rs].float(), torch.full((9,), 5)).to(dtype)
        assert torch.equal(k[ms[6:]], expect)
    # block := old block + old block
    doubled_copy = O.merge_blocks(layers, right, right, alloc, rope)
    O.append_block(layers, right, right, alloc, rope)
    assert right.num_tokens == 18 and right.mrope_span == 18
    ds, rs2 = torch.tensor(doubled_copy.token_slots()), torch.tensor(right.token_slots())
    for k, v in layers:
        assert torch.equal(k[ds], k[rs2]) and torch.equal(v[ds], v[rs2])


def test_zero_shift_is_a_plain_copy_and_shifts_compose():
    rotary, Hkv, D = 16, 2, 16
    g = torch.Generator().manual_seed(7)
    rope = O.RopeSpec(rotary, O.build_cos_sin_cache(rotary, 64, BASE))
    k = torch.randn(40, Hkv, D, generator=g)
    v = torch.randn(40, Hkv, D, generator=g)
    k0, v0 = k.clone(), v.clone()
    O.copy_shift_kv(k, v, [0, 1, 2], [10, 11, 12], 0, rope)
    assert torch.equal(k[10:13], k0[0:3]) and torch.equal(v[10:13], v0[0:3])
    # shifting by 3 and then by 4 lands where a shift by 7 does (rotations add)
    O.copy_shift_kv(k, v, [0, 1, 2], [20, 21, 22], 3, rope)
    O.copy_shift_kv(k, v, [20, 21, 22], [30, 31, 32], 4, rope)
    O.copy_shift_kv(k, v, [0, 1, 2], [33, 34, 35], 7, rope)
    torch.testing.assert_close(k[30:33], k[33:36], atol=1e-5, rtol=1e-5)
    assert torch.equal(v[30:33], v0[0:3])


# ---------------------------------------------------------------------------
# product host logic (no launch without a GPU)
# ---------------------------------------------------------------------------
def make_ops(page=4):
    from types import SimpleNamespace
    from async_llm_amd.shared_cache import SharedCacheAttention

    cpu = torch.device("cpu")
    layer = torch.zeros(8, page, 2, 16, dtype=torch.bfloat16)
    pool = SimpleNamespace(k_cache=lambda _: layer, v_cache=lambda _: layer, num_layers=1)
    att = SharedCacheAttention(pool, torch.zeros(64, 16), 8, 2, 16, page, torch.bfloat16, cpu, rotary_dim=16)
    return BlockKVOps(pool, att, Alloc(page, 1))


def test_block_ops_bookkeeping_and_errors_without_a_gpu():
    ops = make_ops()
    cpu = torch.device("cpu")
    empty_l, empty_r = ops.create_block(), ops.create_block()
    empty_l.token_ids, empty_r.token_ids = [], []
    merged = ops.merge_blocks(empty_l, empty_r)  # nothing to copy: no launch
    assert merged.num_tokens == 0 and merged.page_starts == [] and merged.mrope_span_override is None
    assert ops.append_block(empty_l, empty_r) is empty_l
    wrong = CacheBlock(cpu, 16)
    with pytest.raises(ValueError, match="page size"):
        ops.merge_blocks(wrong, empty_l)
    b = ops.create_block()
    b.grow_pages(ops.page_allocator.alloc_pages(2), 6)
    assert token_slots(b).tolist() == [4, 5, 6, 7, 8, 9]
    with pytest.raises(ValueError, match="overlap"):
        ops._copy_slots([9, 20], b, destination_start=4)
    with pytest.raises(native.ViewAttnError, match="GPU only"):
        ops.merge_blocks(b, empty_r)
