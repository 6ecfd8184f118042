"""Fixed-capacity plans without a GPU: the header (what ``va_attention`` derives
its launches from) depends on the capacity alone, padded plans still cover every
(query sub-row, visible key) pair once, the per-die padding never pushes a plan
that fits over its capacity, and the buffer classes keep the reference's
geometry and capacity errors (reference ``attention_graph.py:74-92, 196-201,
250-252``; its replay test is ``tests/core/test_shared_decode_attention_graph.py``)."""

import random
from types import SimpleNamespace

import numpy as np
import pytest
import torch

from async_llm_amd import native
from async_llm_amd.shared_cache import CacheBlock, PrefillSpec, SharedCacheAttention, WorkerGroup
from async_llm_amd.shared_cache.session_planning import plan_decode_writes
from async_llm_amd.shared_cache.attention_graph import SharedDecodeAttentionBuffers, SharedPrefillAttentionBuffers
from tests.test_native_abi_cpu import H, check_coverage, decode_plan, random_tables

CPU = torch.device("cpu")


def fixed_plan(tables, limits, heads=(8, 2, 64), page=4, dtype=native.VA_BF16, kernel=native.VA_KERNEL_AUTO,
               target=0, capacity=None):
    qo, kvp, kvi, lens, flags, chain, sub_worker, n_rows = tables
    arr = [np.ascontiguousarray(a, dtype=np.int32) for a in (qo, kvp, kvi, lens, flags, chain)]
    sw = np.ascontiguousarray(sub_worker, dtype=np.int64)
    subs = native.VaSubRequests(len(lens), len(sw), n_rows, arr[0].ctypes.data, arr[1].ctypes.data,
                                arr[2].ctypes.data if arr[2].size else None, arr[3].ctypes.data,
                                arr[4].ctypes.data, arr[5].ctypes.data, sw.ctypes.data if sw.size else None)
    shape = native.VaShape(heads[0], heads[1], heads[2], page, dtype)
    params = native.VaPlanParams(kernel, 0, 0, target, 0)
    if capacity is None:
        capacity = native.VaPlanCapacity()
        assert native.lib.va_plan_capacity(shape, params, limits, capacity) == 0, native.lib.va_last_error()
    words = native.lib.va_plan_fixed_words(capacity)
    blob = np.full(words, -7, dtype=np.int32)
    counts = native.VaPlanCounts()
    rc = native.lib.va_plan_build_fixed(subs, shape, params, capacity, blob.ctypes.data, blob.size, counts)
    return rc, blob, counts, capacity


@pytest.mark.parametrize("prefill", [False, True])
@pytest.mark.parametrize("kernel,dtype", [(native.VA_KERNEL_GENERIC, native.VA_F32), (native.VA_KERNEL_MFMA, native.VA_BF16)])
def test_fixed_plans_share_one_header_and_cover_every_pair_once(prefill, kernel, dtype):
    # limits that hold for everything random_tables draws
    limits = native.VaPlanLimits(0, 0, 3, 4, 210, 210) if prefill else native.VaPlanLimits(36, 36, 0, 0, 0, 11)
    headers = []
    for seed in range(10):
        rng = random.Random(300 + seed)
        page = 4
        tables = random_tables(rng, page, prefill)
        qo, kvp, kvi, lens, flags, chain, sub_worker, n_rows = tables
        rc, blob, counts, cap = fixed_plan(tables, limits, page=page, kernel=kernel, dtype=dtype)
        assert rc == 0, native.lib.va_last_error()
        h, items, links, qrefs, indptr, ids, rflags = decode_plan(blob)
        headers.append(h.copy())
        assert h[H["N_ROWS"]] == limits.max_rows and h[H["N_ITEMS"]] == cap.max_items + cap.max_wide_items
        assert h[H["N_WIDE"]] == cap.max_wide_items and h[H["N_PARTIALS"]] == cap.max_partials
        assert counts.workspace_bytes == cap.max_partials * 8 * (64 + 2) * 4
        assert all(int(f) == 2 for f in rflags[n_rows:])  # rows beyond the plan's own: out = 0
        assert all(indptr[r] == indptr[n_rows] for r in range(n_rows, limits.max_rows + 1))
        check_coverage(blob, qo, kvp, lens, flags, sub_worker, n_rows, fixed=True)
    assert all(np.array_equal(h, headers[0]) for h in headers)


@pytest.mark.parametrize("heads", [(16, 4, 256), (4, 2, 64), (8, 8, 128), (4, 1, 64)])
def test_capacity_holds_chains_packed_in_bundles(heads):
    """Prefill chunks of a few wide tiles over views of several thousand tokens: the planner packs
    their tiles in bundles (the slots of a die walk a bundle's tokens side by side; a chain's last
    bundle of few tiles is walked in parts), which makes more items, links and partial states than
    one per tile.  The capacity computed from the limits alone must hold every such plan, and the
    plan must cover every visible pair once."""
    rng = random.Random(heads[0] * 100 + heads[1])
    for case in range(6):
        page = rng.choice([16, 4])
        target = rng.choice([0, 0, 8, 64])
        qo, kvp, kvi, lens, flags, chain, sw = [0], [0], [], [], [], [], []
        n_rows, n_chains, members = 0, rng.randint(1, 5), 1
        for r in range(n_chains):
            new_tokens = rng.choice([1, 9, 33, 64, 65, 138, 300])
            rows = list(range(n_rows, n_rows + new_tokens))
            n_rows += new_tokens
            context = [rng.choice([5, 100, 700, 1500, 4000]) for _ in range(rng.randint(0, 3))]
            members = max(members, len(context) + 1)
            for length in context + [rng.choice([0, 7, 100]) + new_tokens]:
                kvi += list(range(len(kvi), len(kvi) + -(-length // page)))
                kvp.append(len(kvi)); lens.append(length); chain.append(r)
                flags.append(0)
                sw += rows; qo.append(len(sw))
            flags[-1] = 1  # the chunk's own block is the causal one
        limits = native.VaPlanLimits(0, 0, n_chains, members, n_rows, n_rows)
        rc, blob, counts, cap = fixed_plan((qo, kvp, kvi, lens, flags, chain, sw, n_rows), limits, heads=heads, page=page,
                                           dtype=native.VA_BF16, kernel=native.VA_KERNEL_MFMA, target=target)
        assert rc == 0, (case, native.lib.va_last_error())
        check_coverage(blob, qo, kvp, lens, flags, sw, n_rows, fixed=True)


@pytest.mark.parametrize("heads", [(32, 8, 128), (16, 4, 256)])
@pytest.mark.parametrize("target", [0, 1, 8, 16])
def test_capacity_holds_one_row_chunks_over_long_views_beside_a_short_wide_chunk(heads, target):
    """A short wide chunk next to chunks of one new token over long views: the budget that cuts the
    narrow tiles' walks must follow THEIR tokens.  Sized from the wide chunk's few tokens it cut
    every long walk into pieces of the minimum size -- hundreds of items where the capacity derived
    from the limits (narrow items <= chains + target) has room for a few dozen."""
    page = 16
    chains_spec = [(64, [5])] + [(1, [30000] * 4)] * 4
    qo, kvp, kvi, lens, flags, chain, sw = [0], [0], [], [], [], [], []
    n_rows, members = 0, 1
    for r, (new_tokens, context) in enumerate(chains_spec):
        rows = list(range(n_rows, n_rows + new_tokens))
        n_rows += new_tokens
        members = max(members, len(context) + 1)
        for length in context + [new_tokens]:
            kvi += list(range(len(kvi), len(kvi) + -(-length // page)))
            kvp.append(len(kvi)); lens.append(length); chain.append(r); flags.append(0)
            sw += rows; qo.append(len(sw))
        flags[-1] = 1
    tables = (qo, kvp, kvi, lens, flags, chain, sw, n_rows)
    limits = native.VaPlanLimits(0, 0, len(chains_spec), members, n_rows, n_rows)
    rc, blob, counts, cap = fixed_plan(tables, limits, heads=heads, page=page, dtype=native.VA_BF16,
                                       kernel=native.VA_KERNEL_MFMA, target=target)
    assert rc == 0, native.lib.va_last_error()
    check_coverage(blob, qo, kvp, lens, flags, sw, n_rows, fixed=True)
    # the packed plan of the same tables keeps to the same bound: no row with thousands of states
    arr = [np.ascontiguousarray(a, dtype=np.int32) for a in (qo, kvp, kvi, lens, flags, chain)]
    swa = np.ascontiguousarray(sw, dtype=np.int64)
    subs = native.VaSubRequests(len(lens), len(swa), n_rows, arr[0].ctypes.data, arr[1].ctypes.data, arr[2].ctypes.data,
                                arr[3].ctypes.data, arr[4].ctypes.data, arr[5].ctypes.data, swa.ctypes.data)
    packed = native.VaPlanCounts()
    assert native.lib.va_plan_count(subs, native.VaShape(heads[0], heads[1], heads[2], page, native.VA_BF16),
                                    native.VaPlanParams(native.VA_KERNEL_MFMA, 0, 0, target, 0), packed) == 0
    assert packed.n_items - packed.n_wide_items <= cap.max_items


def test_padding_per_die_never_exceeds_a_capacity_the_real_items_fit():
    """One heavy unit and many light ones: dealing by load alone gives one die few
    entries and the others many, and padding every die to the longest list would
    need far more than the real item count.  With a capacity the lists are cut
    at capacity / 8 entries per die."""
    page = 16
    qo, kvp, kvi, lens, flags, chain, sw = [0], [0], [], [], [], [], []
    def add(n_tokens, first_page, w):
        kvi.extend(range(first_page, first_page + -(-n_tokens // page)))
        kvp.append(len(kvi)); lens.append(n_tokens); flags.append(0); chain.append(-1); sw.append(w); qo.append(len(sw))
    add(64, 0, 0)  # one granule: a run this short is never cut
    for w in range(1, 40):
        add(16, 100 + w, w)
    tables = (qo, kvp, kvi, lens, flags, chain, sw, 40)
    limits = native.VaPlanLimits(40, 40, 0, 0, 0, 40)
    rc, blob, counts, cap = fixed_plan(tables, limits, page=page)
    assert rc == 0
    tight = native.VaPlanCapacity(40, 0, cap.max_links, cap.max_qrefs, cap.max_partials, cap.max_row_parts, 40)
    rc, blob, counts, _ = fixed_plan(tables, limits, page=page, capacity=tight)
    assert rc == 0, native.lib.va_last_error()
    h, items, *_ = decode_plan(blob)
    assert h[H["N_ITEMS"]] == 40 and sum(1 for it in items if it[2]) == 40
    check_coverage(blob, qo, kvp, lens, flags, sw, 40, fixed=True)
    short = native.VaPlanCapacity(32, 0, cap.max_links, cap.max_qrefs, cap.max_partials, cap.max_row_parts, 40)
    rc, *_ = fixed_plan(tables, limits, page=page, capacity=short)
    assert rc == native.VA_ERR_CAPACITY and b"work items" in native.lib.va_last_error()
    odd = native.VaPlanCapacity(36, 0, cap.max_links, cap.max_qrefs, cap.max_partials, cap.max_row_parts, 40)
    rc, *_ = fixed_plan(tables, limits, page=page, capacity=odd)
    assert rc == native.VA_ERR_ARG


def test_capacity_refuses_a_pinned_chunk_and_bad_limits():
    shape = native.VaShape(8, 2, 64, 16, native.VA_BF16)
    cap = native.VaPlanCapacity()
    limits = native.VaPlanLimits(8, 8, 0, 0, 0, 4)
    assert native.lib.va_plan_capacity(shape, native.VaPlanParams(0, 0, 512, 0, 0), limits, cap) == native.VA_ERR_ARG
    assert native.lib.va_plan_capacity(shape, native.VaPlanParams(0, 0, 0, 0, 0),
                                       native.VaPlanLimits(8, 4, 0, 0, 0, 4), cap) == native.VA_ERR_ARG
    assert native.lib.va_plan_capacity(shape, native.VaPlanParams(0, 0, 0, 0, 0), limits, cap) == 0
    assert cap.max_items % 8 == 0 and cap.max_wide_items == 0 and cap.max_rows == 4 and cap.max_qrefs == 8


# ---------------------------------------------------------------------------
# the buffer classes (host logic; the tables live on the CPU here)
# ---------------------------------------------------------------------------
def make_attention(page=4, mrope=None):
    pool = SimpleNamespace(k_cache=lambda layer: None, v_cache=lambda layer: None)
    return SharedCacheAttention(pool, torch.zeros(64, 16), 8, 2, 16, page, torch.bfloat16, CPU, rotary_dim=16,
                                mrope_section=mrope, rope_base=10000.0 if mrope else None)


class Pages:
    def __init__(self, page):
        self.page, self.next = page, 1

    def take(self, n):
        got = [(self.next + i) * self.page for i in range(n)]
        self.next += n
        return got

    def alloc_pages(self, n):
        return torch.tensor(self.take(n), dtype=torch.int32)

    def block(self, length, span=None):
        b = CacheBlock(CPU, self.page)
        if length:
            b.grow_pages(torch.tensor(self.take(-(-length // self.page)), dtype=torch.int32), length)
        if span is not None:
            b.mrope_span_override = span
        return b


def test_decode_buffers_keep_the_reference_geometry():
    page = 4
    att = make_attention(page)
    pages = Pages(page)
    a, b, c, own = pages.block(9), pages.block(4), pages.block(0), pages.block(2)
    group = WorkerGroup(cache_structure=[[a, b], [b, c, a], [a]], write_to=[b, a, own])
    pending, slots, _ = plan_decode_writes(group, page, pages, CPU)  # b is full: it opens a page
    buffers = SharedDecodeAttentionBuffers(att, workers=4, depth=3, max_pages=32,
                                           dummy_slots=torch.tensor([900, 901, 902, 903]))
    empty_header = buffers.header.copy()
    meta = att.prepare(group, pending, slots, graph_buffers=buffers)
    plain = att.prepare(group, pending, slots)
    assert meta is buffers.meta and meta.graph_buffers is buffers
    assert meta.num_workers == 4 and meta.max_segments == 4 and meta.n_main == 12 and meta.n_aux == 4
    assert meta.sub_worker.tolist() == [0] * 3 + [1] * 3 + [2] * 3 + [3] * 3 + [0, 1, 2, 3]
    assert meta.pad_slot.tolist() == [0, 1, 2, 4, 5, 6, 8, 9, 10, 12, 13, 14, 3, 7, 11, 15]
    valid = buffers.valid.tolist()
    # every (worker, segment) of the packed plan sits at worker * depth + segment; the writer
    # outside its view (worker 2) at 12 + 2
    expect = {}
    for w, slot, loc in zip(plain.sub_worker.tolist(), plain.pad_slot.tolist(), plain.sub_loc.tolist()):
        seg = slot - w * plain.max_segments
        at = 12 + w if (w == 2 and seg == 1) else w * 3 + seg
        expect[at] = loc
    assert sorted(expect) == [i for i, v in enumerate(valid) if v]
    assert all(meta.sub_loc[i].item() == loc for i, loc in expect.items())
    assert np.array_equal(meta.launch.header, empty_header)
    # the slot table: real token slot for worker 2, dummies elsewhere
    n_entries = 3 * 3 + 2 * 2  # a (3 pages) in three views, b (1 page + the one it opens) in two
    assert buffers._kv_host[n_entries:n_entries + 4].tolist() == [900, 901, slots[2].item(), 903]
    # the padded plan walks the same (sub-row, key) pairs as the packed one
    h, items, links, *_ = decode_plan(buffers._blob_host.numpy())
    packed = decode_plan(plain.launch.blob.numpy())
    assert sorted(int(i[4]) for i in items if i[2]) == sorted(int(i[4]) for i in packed[1] if i[2])
    assert buffers.workspace_requirements() == [(buffers, buffers.counts.workspace_bytes, 0)]


def test_decode_buffers_capacity_errors():
    page = 4
    att = make_attention(page)
    pages = Pages(page)
    blocks = [pages.block(5) for _ in range(4)]
    buffers = SharedDecodeAttentionBuffers(att, workers=2, depth=3, max_pages=6)

    def prepare(views, targets):
        group = WorkerGroup(cache_structure=views, write_to=targets)
        pending, slots, _ = plan_decode_writes(group, page, pages, CPU)
        return att.prepare(group, pending, slots, graph_buffers=buffers)

    with pytest.raises(ValueError, match="Shared attention exceeds graph segment capacity"):
        prepare([blocks], [blocks[0]])
    with pytest.raises(ValueError, match="Shared attention exceeds graph page-index capacity"):
        prepare([blocks[:3], blocks[:3]], [blocks[0], blocks[1]])
    with pytest.raises(ValueError, match="Shared attention exceeds graph worker capacity"):
        prepare([[blocks[0]]] * 3, blocks[1:4])
    # a plan that fits still works afterwards, with the same launch geometry
    meta = prepare([blocks[:1]], [blocks[0]])
    assert buffers.valid.tolist() == [True, False, False, False, False, False, False, False]
    assert meta.sub_loc.tolist()[0] == 5


@pytest.mark.parametrize("mrope", [None, (2, 3, 3)])
def test_prefill_buffers_keep_the_reference_geometry(mrope):
    page = 4
    att = make_attention(page, mrope)
    pages = Pages(page)
    c0, c1 = pages.block(9), pages.block(3, span=2 if mrope else None)
    rel = torch.tensor([[0, 1, 1, 2, 3], [0, 1, 2, 2, 3], [0, 1, 1, 1, 3]]) if mrope else None
    specs = [
        PrefillSpec([c0, c1], torch.tensor(pages.take(2)), 6, 0),
        PrefillSpec([c1], torch.tensor(pages.take(2)), 5, 3, 2 if mrope else None, rel),
        PrefillSpec([], torch.tensor(pages.take(1)), 2, 1),
    ]
    buffers = SharedPrefillAttentionBuffers(att, workers=4, depth=2, rows=16, max_pages=20)
    empty_header = buffers.header.copy()
    meta = att.prepare_prefill_batch(specs, graph_buffers=buffers)
    plain = att.prepare_prefill_batch(specs)
    assert meta is buffers.meta and np.array_equal(meta.launch.header, empty_header)
    assert meta.num_workers == 16 and meta.max_segments == 3 and meta.n_ctx_rows == 32
    n_ctx, n_new = 6 * 2 + 5, 13
    assert buffers.used_ctx_rows == n_ctx and buffers.used_self_rows == n_new
    assert meta.last_indices.tolist() == [5, 10, 12, 0] and plain.last_indices.tolist() == [5, 10, 12]
    # context sub-rows first (as the packed plan orders them), self sub-rows at their fixed place
    assert meta.sub_worker[:n_ctx].tolist() == plain.sub_worker[:n_ctx].tolist()
    assert meta.sub_worker[32:].tolist() == list(range(16))
    assert torch.equal(meta.sub_loc[..., :n_ctx], plain.sub_loc[..., :n_ctx])
    assert torch.equal(meta.sub_loc[..., 32:32 + n_new], plain.sub_loc[..., n_ctx:])
    assert meta.pad_slot[:n_ctx].tolist() == plain.pad_slot[:n_ctx].tolist()
    assert meta.pad_slot[32:32 + n_new].tolist() == plain.pad_slot[n_ctx:].tolist()
    assert sorted(meta.pad_slot.tolist()) == list(range(48))  # a permutation, padding included
    assert buffers.valid.tolist() == [True] * n_ctx + [False] * (32 - n_ctx) + [True] * n_new + [False] * 3
    h, items, links, *_ = decode_plan(buffers._blob_host.numpy())
    packed = decode_plan(plain.launch.blob.numpy())
    assert sorted(int(i[4]) for i in items if i[2]) == sorted(int(i[4]) for i in packed[1] if i[2])
    rflags = buffers._blob_host.numpy()[h[H["OFF_ROW_FLAGS"]]: h[H["OFF_ROW_FLAGS"]] + 16]
    assert all(int(f) == 2 for f in rflags[n_new:]) and all(int(f) != 2 for f in rflags[:n_new])


def test_prefill_buffers_capacity_errors():
    page = 4
    att = make_attention(page)
    pages = Pages(page)
    ctx = [pages.block(5) for _ in range(3)]
    buffers = SharedPrefillAttentionBuffers(att, workers=2, depth=2, rows=8, max_pages=5)
    message = "Shared prefill exceeds graph request/row/segment capacity"
    one = lambda n, context=(): PrefillSpec(list(context), torch.tensor(pages.take(-(-n // page))), n, 0)
    with pytest.raises(ValueError, match=message):
        buffers.plan([one(1), one(1), one(1)])
    with pytest.raises(ValueError, match=message):
        buffers.plan([one(5), one(4)])
    with pytest.raises(ValueError, match=message):
        buffers.plan([one(2, ctx)])
    with pytest.raises(ValueError, match="Shared prefill exceeds graph page-index capacity"):
        buffers.plan([one(8, ctx[:2])])
    meta = buffers.plan([one(3, ctx[:1])])
    assert buffers.used_ctx_rows == 3 and buffers.used_self_rows == 3 and meta.last_indices.tolist() == [2, 0]


def test_prepare_workspace_takes_the_largest_profile():
    att = make_attention(4)
    small = SharedDecodeAttentionBuffers(att, workers=2, depth=2, max_pages=8)
    large = SharedPrefillAttentionBuffers(att, workers=2, depth=2, rows=64, max_pages=64)
    need = max(entry[1] for entry in small.workspace_requirements() + large.workspace_requirements())
    assert need == max(large.counts.workspace_bytes, small.counts.workspace_bytes) > 0
    att._workspace = None
    att.prepare_workspace([small, large])
    assert att._workspace.numel() == need
    # both profiles launch out of the one arena
    assert small.meta.launch.workspace is att._workspace and large.meta.launch.workspace is att._workspace
    with pytest.raises(RuntimeError, match="prepared once"):
        att.prepare_workspace([small])
    other = make_attention(4)
    with pytest.raises(ValueError, match="belong to this instance"):
        other.prepare_workspace([small])


def bare_attention(monkeypatch):
    """An op with nothing but its workspace state, as the reference's workspace tests build one
    (``tests/core/test_attention_workspace.py:14-20``)."""
    monkeypatch.setattr(torch.cuda, "is_current_stream_capturing", lambda: False)
    att = SharedCacheAttention.__new__(SharedCacheAttention)
    att.device = CPU
    att._workspace = torch.empty(8, dtype=torch.uint8)
    att._workspace_prepared = False
    return att


@pytest.mark.parametrize("reverse", [False, True])
def test_catalogue_shares_the_largest_arena_but_not_the_table_storage(monkeypatch, reverse):
    # known answers of the reference's tests/core/test_attention_workspace.py:23-41
    att = bare_attention(monkeypatch)
    consumers = [SimpleNamespace() for _ in range(4)]
    for c in consumers:
        def reset(arena, ints, c=c):
            c.arena, c.ints = arena, ints
        c.reset_workspace_buffer = reset
    decode = SimpleNamespace(attention=att, workspace_requirements=lambda: [(consumers[0], 32, 24), (consumers[1], 16, 0)])
    prefill = SimpleNamespace(attention=att, workspace_requirements=lambda: [(consumers[2], 64, 48), (consumers[3], 8, 16)])
    att.prepare_workspace([prefill, decode] if reverse else [decode, prefill])
    assert att._workspace.numel() == 64
    assert all(c.arena is att._workspace for c in consumers)
    assert [c.ints.numel() for c in consumers] == [24, 16, 48, 16]
    assert len({c.ints.data_ptr() for c in consumers}) == 4
    with pytest.raises(RuntimeError, match="once before capture"):
        att.prepare_workspace([decode])


def test_failed_allocation_or_capture_rebinds_nothing(monkeypatch):
    # the scenario of the reference's tests/core/test_attention_workspace.py:44-68: the third
    # allocation (arena, first table, SECOND table) fails
    att = bare_attention(monkeypatch)
    original = att._workspace
    calls = []
    consumer = SimpleNamespace(reset_workspace_buffer=lambda *args: calls.append(args))
    profile = SimpleNamespace(attention=att, workspace_requirements=lambda: [(consumer, 64, 24), (consumer, 32, 48)])
    real_empty, count = torch.empty, 0

    def allocate(*args, **kwargs):
        nonlocal count
        count += 1
        if count == 3:
            raise torch.OutOfMemoryError("test allocation")
        return real_empty(*args, **kwargs)

    with monkeypatch.context() as patch:
        patch.setattr(torch, "empty", allocate)
        with pytest.raises(torch.OutOfMemoryError):
            att.prepare_workspace([profile])
    assert not calls and att._workspace is original and not att._workspace_prepared
    att.device = torch.device("cuda")  # capture is only ever asked about on a GPU op
    monkeypatch.setattr(torch.cuda, "is_current_stream_capturing", lambda: True)
    with pytest.raises(RuntimeError, match="before capture"):
        att.prepare_workspace([profile])
    assert not calls and not att._workspace_prepared


def test_empty_catalogue_and_foreign_owner(monkeypatch):
    att = bare_attention(monkeypatch)
    att.prepare_workspace([])
    assert not att._workspace_prepared
    with pytest.raises(ValueError, match="belong"):
        att.prepare_workspace([SimpleNamespace(attention=object())])
