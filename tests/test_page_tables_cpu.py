"""Integer tables of the planners, bit-exact.

Known answers are those the reference asserts in
tests/core/test_attention_metadata.py (:32-60 snapshots and index table,
:117-148 decode plan, :151-182 prefill plan, :185-201 slot planning) plus the
hand-derived tables of the plumbing configuration; random cases compare the
product planner with the oracle's restatement of the reference planner.
"""

import random
from types import SimpleNamespace

import pytest
import torch

from async_llm_amd.shared_cache import CacheBlock, PrefillSpec, SharedCacheAttention, WorkerGroup
from async_llm_amd.shared_cache.attention_metadata import page_numbers, upload_page_indices
from async_llm_amd.shared_cache.session_planning import alloc_token_storage, plan_decode_writes
from async_llm_amd.kvcache import PageAllocator
from oracle import view_attention_oracle as O
from tests.util import oracle_decode_plan, oracle_prefill_plan

CPU = torch.device("cpu")


class CountedPages(list):
    reads = 0

    def __iter__(self):
        self.reads += 1
        return super().__iter__()


def block(page, pages, length):
    b = CacheBlock(CPU, page)
    b.page_starts = CountedPages([p * page for p in pages])
    b.num_tokens = length
    return b


def make_op(page, heads=(8, 2, 64), dtype=torch.bfloat16, kernel=None):
    return SharedCacheAttention(SimpleNamespace(), torch.zeros(4, heads[2]), heads[0], heads[1], heads[2], page,
                                dtype, CPU, kernel=kernel)


def entries(plan):
    ids = plan.get("indices", plan.get("paged_kv_indices")).tolist()
    off = plan.get("indptr", plan.get("paged_kv_indptr")).tolist()
    return [ids[a:b] for a, b in zip(off, off[1:])]


@pytest.mark.parametrize("page", [1, 4, 16])
def test_snapshot_is_per_prepare_and_includes_pending_page_once(page):
    b = block(page, [7, 2], 2 * page)
    snap = {}
    first = page_numbers(b, snap, 11 * page)
    assert first == [7, 2, 11]
    assert page_numbers(b, snap, 11 * page) is first
    assert b.page_starts.reads == 1
    assert b.page_starts == [7 * page, 2 * page]
    b.append_token(11 * page)
    b.page_starts[0] = 13 * page
    assert page_numbers(b, {}) == [13, 2, 11]
    assert first == [7, 2, 11]
    b.clear()
    assert page_numbers(b, {}) == []
    assert page_numbers(b, {}, 19 * page) == [19]


@pytest.mark.parametrize("parts", [[], [[], []], [[7, 2], [], [7, 2], [11]]])
def test_bulk_index_table_order_empty_and_owners(parts):
    refs = []
    indices = upload_page_indices(parts, CPU, refs)
    assert indices.dtype == torch.int32 and indices.ndim == 1
    assert indices.tolist() == [p for part in parts for p in part]
    assert len(refs) == 2 and refs[1] is indices
    before = indices.clone()
    for part in parts:
        part.clear()
    assert torch.equal(indices, before)


@pytest.mark.parametrize("page", [1, 4, 16])
def test_decode_cross_readers_empty_blocks_duplicates_and_implicit_self(page):
    a = make_op(page)
    common, left, right, empty = (block(page, [7, 2], page + 1), block(page, [11], page),
                                  block(page, [], 0), block(page, [], 0))
    common.mrope_span_override = 1
    group = WorkerGroup(cache_structure=[[common, empty, right, left], [common, left, common]],
                        write_to=[left, right])
    pending = {id(left): 13 * page, id(right): 17 * page}
    meta = a.prepare(group, pending, torch.tensor([13 * page, 17 * page]))
    assert common.page_starts.reads == left.page_starts.reads == right.page_starts.reads == 1
    main, aux = meta.main_plan, meta.aux_plan
    assert entries(main) == [[7, 2], [17], [11, 13], [7, 2], [11, 13], [7, 2]]
    assert main["seq_lens"].tolist() == [page + 1, 1, page + 1, page + 1, page + 1, page + 1]
    assert meta.sub_loc.tolist() == [page + 2, page + 1, page, page + 2, page + 1, 0] + [0]
    assert entries(aux) == [[17 * page]]
    assert aux["seq_lens"].tolist() == [1] and aux["page_size"] == 1
    assert "max_token_per_sequence" not in main
    assert left.page_starts == [11 * page] and right.page_starts == []  # blocks untouched
    assert (meta.n_main, meta.n_aux, meta.max_segments, meta.num_workers) == (6, 1, 4, 2)
    assert meta.sub_worker.tolist() == [0, 0, 0, 1, 1, 1, 1]
    assert meta.pad_slot.tolist() == [0, 1, 2, 4, 5, 6, 7]  # worker * max_segments + segment
    last = main["last_page_len"].tolist()
    assert last == [n - (len(e) - 1) * page for n, e in zip(main["seq_lens"].tolist(), entries(main))]
    assert meta.get_last_indices(2).tolist() == [0, 1]
    # the oracle's restatement of the reference planner agrees table by table
    oplan = oracle_decode_plan(group, pending, torch.tensor([13 * page, 17 * page]), page)
    assert oplan.sub_loc == meta.sub_loc.tolist() and oplan.pad_slot == meta.pad_slot.tolist()
    assert oplan.kv_indices == main["indices"].tolist() and oplan.kv_indptr == main["indptr"].tolist()
    assert oplan.aux_slots == aux["indices"].tolist()


def test_plumbing_configuration_tables():
    """3-block view 256/1024/512, the writer appends to the last block and opens
    page 33 of it: lengths 256/1024/513, rotations 1792/1536/512."""
    P = 16
    a = make_op(P, heads=(8, 2, 128), dtype=torch.float32)
    b0, b1, b2 = block(P, range(0, 16), 256), block(P, range(16, 80), 1024), block(P, range(80, 112), 512)
    group = WorkerGroup(cache_structure=[[b0, b1, b2]])
    alloc = SimpleNamespace(alloc_pages=lambda n: torch.tensor([200 * P]))
    pending, slots, pos = plan_decode_writes(group, P, alloc, CPU)
    assert pending == {id(b2): 200 * P} and slots.tolist() == [200 * P] and pos == [512]
    meta = a.prepare(group, pending, slots)
    assert meta.sub_loc.tolist() == [1792, 1536, 512]
    assert meta.main_plan["seq_lens"].tolist() == [256, 1024, 513]
    assert meta.main_plan["last_page_len"].tolist() == [16, 16, 1]
    assert meta.main_plan["indptr"].tolist() == [0, 16, 80, 113]
    assert meta.main_plan["indices"].tolist()[-1] == 200
    assert meta.sub_worker.tolist() == [0, 0, 0] and meta.pad_slot.tolist() == [0, 1, 2]
    assert (meta.max_segments, meta.n_main, meta.n_aux) == (3, 3, 0)


@pytest.mark.parametrize("context", [False, True])
def test_prefill_tables_track_real_rows(context):
    P = 4
    a = make_op(P)
    shared = block(P, [7, 2], 5)
    shared.mrope_span_override = 2
    for lengths in ([3, 9], [1], [7, 13, 5]):
        shared.page_starts.reads = 0
        specs = [PrefillSpec([shared, shared] if context else [],
                             torch.arange(20 + i * 8, 20 + i * 8 + (2 + n + 3) // 4) * 4, n, 2, 1,
                             torch.arange(n).expand(3, -1)) for i, n in enumerate(lengths)]
        meta = a.prepare_prefill_batch(specs)
        assert shared.page_starts.reads == int(context)
        main, own = meta.main_plan, meta.aux_plan
        for plan in (main, own):
            if plan is None:
                continue
            qlens = plan["qo_indptr"].diff().tolist()
            assert plan["max_token_per_sequence"] == max(qlens)
        assert own["max_token_per_sequence"] == max(lengths)
        assert int(own["qo_indptr"][-1]) == sum(lengths)
        assert entries(own) == [[int(p) // 4 for p in s.self_page_starts] for s in specs]
        assert own["seq_lens"].tolist() == [2 + n for n in lengths] and own["causal"] is True
        if context:
            assert entries(main) == [[7, 2]] * (2 * len(specs))
            assert main["seq_lens"].tolist() == [5] * (2 * len(specs)) and main["causal"] is False
            assert main["paged_kv_last_page_len"].tolist() == [1] * (2 * len(specs))
        else:
            assert main is None and meta.n_ctx_rows == 0
        assert meta.sub_loc.shape[0] == 3  # one 3-D request forces 3-axis positions
        offs = [sum(lengths[:i]) for i in range(len(lengths))]
        assert meta.last_indices.tolist() == [o + n - 1 for o, n in zip(offs, lengths)]
        assert meta.phase == "prefill_batch" and meta.get_last_indices(0) is meta.last_indices
        assert len(set(meta.pad_slot.tolist())) == meta.pad_slot.numel()  # injective scatter
        oplan = oracle_prefill_plan(specs, P)
        assert torch.equal(oplan.sub_loc, meta.sub_loc) and oplan.pad_slot == meta.pad_slot.tolist()
        assert oplan.sub_worker == meta.sub_worker.tolist() and oplan.n_ctx_rows == meta.n_ctx_rows
        shared.page_starts = CountedPages([28, 8])


def test_prefill_worked_example():
    """First request of lengths [3, 9] with context [shared, shared]: shared has 5
    tokens, span 2; the write block already holds 2 tokens with span 1."""
    P = 4
    a = make_op(P)
    shared = block(P, [7, 2], 5)
    shared.mrope_span_override = 2
    spec = PrefillSpec([shared, shared], torch.tensor([80, 84]), 3, 2, 1, torch.arange(3).expand(3, -1))
    meta = a.prepare_prefill_batch([spec])
    assert meta.sub_loc[0].tolist() == [5, 6, 7, 3, 4, 5, 1, 2, 3]
    assert meta.sub_worker.tolist() == [0, 1, 2] * 3
    assert meta.pad_slot.tolist() == [0, 3, 6, 1, 4, 7, 2, 5, 8]
    assert entries(meta.aux_plan) == [[20, 21]] and meta.aux_plan["paged_kv_last_page_len"].tolist() == [1]
    assert (meta.max_segments, meta.n_ctx_rows, meta.num_workers) == (3, 6, 3)
    assert meta.last_indices.tolist() == [2]


def test_decode_slot_allocator_uses_one_bulk_readback(monkeypatch):
    page = 4
    a, b, c = block(page, [3], 4), block(page, [8], 2), block(page, [], 0)
    calls = []

    def allocate(n):
        calls.append(n)
        return torch.tensor([40, 52])

    def no_scalar(*args):
        raise AssertionError("per-slot scalar readback")

    monkeypatch.setattr(torch.Tensor, "item", no_scalar)
    pending, slots, positions = plan_decode_writes(WorkerGroup(cache_structure=[[a], [b], [c]]), page,
                                                   SimpleNamespace(alloc_pages=allocate), CPU)
    assert calls == [2] and pending == {id(a): 40, id(b): None, id(c): 52}
    assert slots.tolist() == [40, 34, 52] and positions == [4, 2, 0]
    assert slots.dtype == torch.int32


def test_alloc_token_storage_fills_tail_first():
    alloc = PageAllocator(16, 4, CPU)
    b = CacheBlock(CPU, 4)
    pages, slots = alloc_token_storage(5, 4, alloc, CPU, b)
    assert pages.tolist() == [0, 4] and slots.tolist() == [0, 1, 2, 3, 4]
    b.grow_pages(pages, 5)
    pages, slots = alloc_token_storage(6, 4, alloc, CPU, b)
    assert pages.tolist() == [8] and slots.tolist() == [5, 6, 7, 8, 9, 10]
    assert alloc.num_free_pages == 13
    alloc.free_pages(torch.tensor([0, 4, 8]))
    assert alloc.num_free_pages == 16
    with pytest.raises(RuntimeError, match="out of pages"):
        alloc.alloc_pages(17)


@pytest.mark.parametrize("seed", range(6))
def test_random_decode_plans_match_oracle(seed):
    rng = random.Random(seed)
    P = rng.choice([1, 4, 16])
    a = make_op(P)
    next_page = [0]

    def fresh(n_tokens, span=None):
        b = CacheBlock(CPU, P)
        pages = -(-n_tokens // P)
        b.page_starts = [(next_page[0] + i) * P for i in range(pages)]
        next_page[0] += pages
        b.num_tokens = n_tokens
        if span is not None:
            b.mrope_span_override = span
        return b

    shared = [fresh(rng.randint(0, 40), rng.choice([None, 3])) for _ in range(4)]
    W = rng.randint(1, 6)
    own = [fresh(rng.randint(0, 3 * P)) for _ in range(W)]
    views = []
    for w in range(W):
        view = rng.sample(shared, rng.randint(0, 4)) + rng.sample(own, rng.randint(0, min(3, W)))
        rng.shuffle(view)
        if rng.random() < 0.7 and own[w] not in view:
            view.append(own[w])
        if rng.random() < 0.3 and view:
            view.append(view[0])  # a block may appear twice in one view
        views.append(view or [own[w]])
    group = WorkerGroup(cache_structure=views, write_to=own)
    alloc = SimpleNamespace(alloc_pages=lambda n: torch.arange(1000, 1000 + n) * P)
    pending, slots, _ = plan_decode_writes(group, P, alloc, CPU)
    meta = a.prepare(group, pending, slots)
    oplan = oracle_decode_plan(group, pending, slots, P)
    assert meta.sub_worker.tolist() == oplan.sub_worker
    assert meta.sub_loc.tolist() == oplan.sub_loc
    assert meta.pad_slot.tolist() == oplan.pad_slot
    assert (meta.n_main, meta.n_aux, meta.max_segments) == (oplan.n_main, oplan.n_aux, oplan.max_segments)
    if meta.n_main:
        assert meta.main_plan["indptr"].tolist() == oplan.kv_indptr
        assert meta.main_plan["indices"].tolist() == oplan.kv_indices
        assert meta.main_plan["seq_lens"].tolist() == oplan.seq_lens
        assert meta.main_plan["last_page_len"].tolist() == oplan.last_page_len
    if meta.n_aux:
        assert meta.aux_plan["indices"].tolist() == oplan.aux_slots
    assert meta.main_plan is None or meta.main_plan["indices"].dtype == torch.int32


def test_prepare_rejects_bad_input():
    a = make_op(4)
    with pytest.raises(AssertionError):
        a.prepare_prefill_batch([])
    empty = CacheBlock(CPU, 4)
    with pytest.raises(AssertionError, match="non-empty"):
        a.prepare_prefill_batch([PrefillSpec([empty], torch.tensor([0]), 2)])
    with pytest.raises(AssertionError, match="mrope_rel"):
        a.prepare_prefill_batch([PrefillSpec([], torch.tensor([0]), 2, mrope_rel=torch.zeros(3, 5))])
    with pytest.raises(ValueError, match="kernel"):
        make_op(4, kernel="cuda")


def test_page_array_cache_follows_every_change_of_the_page_list():
    """The planners keep each block's page numbers as an array between prepares;
    the array must equal the list-built table after every kind of change a
    session makes to a block (reference shared_block.py grow/append/clear,
    session.py:352 assignment), and foreign block objects are never cached."""
    from async_llm_amd.shared_cache.attention_metadata import page_array, page_numbers_array

    page = 4
    b = CacheBlock(torch.device("cpu"), page)

    def check():
        want = page_numbers(b, {})
        got = page_array(b)
        assert got.dtype.name == "int32" and got.tolist() == want
        assert page_numbers_array(b, {}, 40).tolist() == want + [10]
        assert page_array(b) is got  # served from the cache while nothing changes

    check()
    b.grow_pages(torch.tensor([8, 20]), 7)
    check()
    b.append_token(None)
    check()
    b.append_token(32)  # opens a page
    check()
    b.page_starts = [4, 12, 16]  # a session assigning a fresh list (merge)
    b.num_tokens = 12
    check()
    b.page_starts = [4, 12, 36]  # same length, different content
    check()
    b.clear()
    check()
    b.grow_pages(torch.tensor([4, 12, 36]), 9)
    check()
    foreign = SimpleNamespace(page_starts=[8, 4], page_size=page)
    first = page_array(foreign)
    foreign.page_starts[0] = 16  # changed in place, no version counter: must be seen
    assert first.tolist() == [2, 1] and page_array(foreign).tolist() == [4, 1]
