"""Block / context / group arithmetic.  Known answers transcribed from the
reference's CPU tests (tests/core/test_shared_cache.py:50-175,
tests/core/test_async_cache_primitives.py)."""

import pytest
import torch

from async_llm_amd.shared_cache import AsyncContext, CacheBlock, SharedBlock, WorkerGroup

CPU = torch.device("cpu")


def filled(n, first_page=0, page_size=1):
    b = CacheBlock(CPU, page_size=page_size)
    pages = -(-n // page_size)
    b.grow_pages(torch.arange(first_page, first_page + pages, dtype=torch.int32) * page_size, n)
    return b


def test_alias_and_ids():
    assert SharedBlock is CacheBlock
    assert CacheBlock(CPU).block_id != CacheBlock(CPU).block_id


def test_empty_block():
    b = SharedBlock(CPU)
    assert (b.num_tokens, b.num_pages, b.last_page_len, b.has_capacity, b.free_tail) == (0, 0, 0, False, 0)
    assert b.token_slots_tensor().tolist() == []


def test_grow_page_size_1_and_4():
    b = SharedBlock(CPU, page_size=1)
    b.grow_pages(torch.tensor([10, 11, 12], dtype=torch.int32), 3)
    assert b.page_starts == [10, 11, 12] and b.num_tokens == 3
    assert b.token_slots_tensor().tolist() == [10, 11, 12]
    assert b.page_numbers_tensor().tolist() == [10, 11, 12]
    b = SharedBlock(CPU, page_size=4)
    b.grow_pages(torch.tensor([0, 4], dtype=torch.int32), 5)
    assert (b.num_tokens, b.num_pages, b.last_page_len, b.has_capacity) == (5, 2, 1, True)
    assert b.token_slots_tensor().tolist() == [0, 1, 2, 3, 4]
    assert b.page_numbers_tensor().tolist() == [0, 1]


def test_append_token_growth():
    b = SharedBlock(CPU, page_size=4)
    b.grow_pages(torch.tensor([0, 4], dtype=torch.int32), 5)
    b.append_token(None)
    assert b.num_tokens == 6 and b.last_page_len == 2
    b.append_token(None)
    b.append_token(None)
    assert b.num_tokens == 8 and not b.has_capacity
    with pytest.raises(AssertionError):
        b.append_token(None)
    b.append_token(8)
    assert b.page_starts == [0, 4, 8] and b.last_page_len == 1
    assert b.token_slots_tensor().tolist() == list(range(9))
    with pytest.raises(AssertionError):
        b.append_token(12)


def test_pages_needed_and_extend():
    b = SharedBlock(CPU, page_size=4)
    assert b.free_tail == 0 and b.pages_needed(1) == 1 and b.pages_needed(9) == 3
    b.grow_pages(torch.tensor([0, 4], dtype=torch.int32), 5)
    assert b.free_tail == 3
    assert [b.pages_needed(n) for n in (3, 4, 12)] == [0, 1, 3]
    b.grow_pages(torch.tensor([], dtype=torch.int32), 3)
    assert b.num_tokens == 8 and b.page_starts == [0, 4] and not b.has_capacity
    b.grow_pages(torch.tensor([8, 12], dtype=torch.int32), 5)
    assert b.num_tokens == 13 and b.page_starts == [0, 4, 8, 12] and b.last_page_len == 1
    with pytest.raises(AssertionError, match="grow_pages got"):
        b.grow_pages(torch.tensor([16], dtype=torch.int32), 2)


def test_clear_and_span():
    b = SharedBlock(CPU, page_size=4)
    b.grow_pages(torch.tensor([8, 12], dtype=torch.int32), 6)
    b.token_ids.extend([1, 2, 3])
    b.mrope_span_override = 3
    assert b.mrope_span == 3
    b.append_token(None)
    assert b.mrope_span == 4 and b.num_tokens == 7  # decoded tokens advance the span too
    b.linear_affine[0] = (torch.zeros(1), torch.zeros(1))
    b._gdn_state_cache.prepared = object()
    assert b.clear() == [8, 12]
    assert b.num_tokens == 0 and b.num_pages == 0 and b.token_ids == [] and b.mrope_span == 0
    assert b._gdn_state_cache.prepared is None and len(b.linear_affine) == 0


def test_state_dict_invalidates_on_mutation():
    b = SharedBlock(CPU)
    for mutate in (lambda d: d.__setitem__(1, 2), lambda d: d.update({3: 4}), lambda d: d.pop(1),
                   lambda d: d.setdefault(9, 1), lambda d: d.clear()):
        b._gdn_state_cache.prepared = "ready"
        mutate(b.linear_conv_state)
        assert b._gdn_state_cache.prepared is None


def test_async_context():
    a, b = filled(2), filled(3, first_page=2)
    ctx = AsyncContext(cache_view=[a, b])
    assert ctx.output_block is b and ctx.num_cached_tokens == 5
    out = CacheBlock(CPU)
    ctx = AsyncContext(cache_view=[a], output_block=out)
    assert ctx.output_block is out and ctx.num_cached_tokens == 2
    with pytest.raises(AssertionError):
        AsyncContext(cache_view=[])


def test_worker_group_forms():
    prompt, w1, w2 = filled(4), filled(2, 4), filled(3, 6)
    group = WorkerGroup([AsyncContext(cache_view=[prompt, w2, w1]), AsyncContext(cache_view=[prompt, w1, w2])])
    assert group.num_workers == 2 and len(group) == 2
    assert group.cache_structure == [[prompt, w2, w1], [prompt, w1, w2]]
    assert group.write_to == [w1, w2]
    assert group.worker_cache_length(0) == 9 and group.max_cache_length() == 9
    legacy = WorkerGroup(cache_structure=[[prompt, w2, w1], [prompt, w1, w2]], write_to=[w1, w2])
    assert legacy.cache_structure == group.cache_structure and legacy.write_to == [w1, w2]
    a, b, c = filled(1), filled(1, 1), filled(1, 2)
    assert WorkerGroup(cache_structure=[[a, b], [a, c]]).write_to == [b, c]
    assert isinstance(group[0], AsyncContext) and group[1].output_block is w2
    tail = group[1:]
    assert isinstance(tail, WorkerGroup) and tail.write_to == [w2]
    assert [ctx.output_block for ctx in group] == [w1, w2]


def test_worker_group_rejections():
    prompt, w = filled(2), filled(1, first_page=2)
    with pytest.raises(ValueError, match="writing the same block"):
        WorkerGroup([AsyncContext(cache_view=[prompt, w]), AsyncContext(cache_view=[w])])
    ctx = AsyncContext(cache_view=[prompt])
    with pytest.raises(AssertionError):
        WorkerGroup([ctx], cache_structure=[[prompt]])
    with pytest.raises(AssertionError):
        WorkerGroup()


def test_op_refuses_a_pool_whose_layers_are_not_plain_paged_arrays():
    """The op writes K/V rows into the pool itself (the reference calls ``kv_cache.store_kv``,
    ``attention.py:649``), so the layout it assumes is checked when it is built."""
    from types import SimpleNamespace

    import pytest

    from async_llm_amd.shared_cache import SharedCacheAttention

    def build(layer, dtype=torch.bfloat16):
        pool = SimpleNamespace(k_cache=lambda _: layer, v_cache=lambda _: layer)
        return SharedCacheAttention(pool, torch.zeros(64, 16), 8, 2, 16, 4, dtype, torch.device("cpu"), rotary_dim=16)

    build(torch.zeros(8, 4, 2, 16, dtype=torch.bfloat16))
    with pytest.raises(ValueError, match="must be"):
        build(torch.zeros(8, 2, 4, 16, dtype=torch.bfloat16))  # heads before tokens
    with pytest.raises(ValueError, match="contiguous"):
        build(torch.zeros(8, 4, 2, 32, dtype=torch.bfloat16)[..., :16])
    with pytest.raises(ValueError, match="contiguous"):
        build(torch.zeros(8, 4, 2, 16, dtype=torch.float16))


def test_get_rope_index_known_answers_and_reference_fixtures():
    """The product's ``get_rope_index`` (reference ``models/qwen3_5_mrope.py:19-64``) against the
    known answers of the reference's ``tests/core/test_qwen3_5_vision_encoder.py:70-92`` and the
    HF-generated position fixtures the reference holds (``tests/resources/qwen3_5_0.8B_ref*.npz``,
    kept here as ``tests/golden/mrope_positions.json``)."""
    import json
    import os

    from async_llm_amd.shared_cache.mrope import get_rope_index

    ids = torch.zeros(5, dtype=torch.int64)
    pos = get_rope_index(ids, torch.zeros(5, dtype=torch.int64), 2)
    assert torch.equal(pos, torch.arange(5).view(1, -1).expand(3, -1))
    kinds = torch.tensor([0, 0, 1, 1, 1, 1, 0, 0, 0])
    pos = get_rope_index(torch.zeros(9, dtype=torch.int64), kinds, 2, torch.tensor([[1, 4, 4]]))
    assert pos.shape == (3, 9)
    assert pos[0].tolist() == [0, 1, 2, 2, 2, 2, 4, 5, 6]
    assert pos[1].tolist() == [0, 1, 2, 2, 3, 3, 4, 5, 6]
    assert pos[2].tolist() == [0, 1, 2, 3, 2, 3, 4, 5, 6]
    with pytest.raises(NotImplementedError):
        get_rope_index(torch.zeros(2, dtype=torch.int64), torch.tensor([0, 7]), 2)
    with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "mrope_positions.json")) as f:
        cases = json.load(f)
    assert cases
    for case in cases:
        kinds = torch.tensor(case["mm_token_type_ids"])
        got = get_rope_index(torch.zeros_like(kinds), kinds, case["spatial_merge_size"],
                             torch.tensor(case["image_grid_thw"]))
        assert got.tolist() == case["rope_positions"], case["source"]


def test_image_block_span_of_the_long_context_workload():
    """The mRoPE decode workload takes its block span from ``get_rope_index``: a 4096-token image
    on a 64 x 64 lattice advances the running position by 64 only."""
    from async_llm_amd.shared_cache.mrope import get_rope_index

    kinds = torch.tensor([0] * 100 + [1] * 4096 + [0] * 50)
    pos = get_rope_index(kinds, kinds, 2, torch.tensor([[1, 128, 128]]))
    assert int(pos.max()) + 1 == 100 + 64 + 50
    assert pos[:, 100].tolist() == [100, 100, 100] and pos[:, 100 + 4095].tolist() == [100, 163, 163]
    assert pos[:, 100 + 4096].tolist() == [164, 164, 164]
