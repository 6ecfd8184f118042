"""GPU parity of view-attention decode: product op (HIP through the C ABI) vs
the CPU oracle on identical seeded inputs.  Scenarios follow the reference's
tests: cross readers, duplicate blocks, empty blocks, writer outside its view
(tests/core/test_attention_metadata.py:117-148), page sizes 1/4/16, partial
rotary and mRoPE (tests/core/test_shared_decode_attention_graph.py:16-107) and
the K=0/V=1 known answer (tests/core/test_attention_workspace.py:79-126)."""

import math
from types import SimpleNamespace

import pytest
import torch

from async_llm_amd import workloads
from async_llm_amd.shared_cache import CacheBlock, SharedCacheAttention, WorkerGroup
from oracle import view_attention_oracle as O
from tests.util import assert_close, make_op_and_pool, oracle_decode_plan, oracle_rope, run_decode_parity

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda")
KERNELS = ["generic", "auto"]


class Pages:
    def __init__(self, page, first=0):
        self.page, self.next = page, first

    def take(self, n):
        got = [(self.next + i) * self.page for i in range(n)]
        self.next += n
        return got

    def alloc_pages(self, n):
        return torch.tensor(self.take(n), dtype=torch.int32)

    def block(self, length, span=None):
        b = CacheBlock(DEV, self.page)
        if length:
            b.grow_pages(torch.tensor(self.take(-(-length // self.page)), dtype=torch.int32), length)
        if span is not None:
            b.mrope_span_override = span
        return b


@pytest.mark.parametrize("kernel", KERNELS)
def test_plumbing_configuration_fp32(kernel):
    """Configuration 1: fp32, 3-block view 256/1024/512, 8 q / 2 kv heads, D 128."""
    wl = workloads.plumbing_decode(DEV, kernel=kernel)
    meta = wl.meta
    assert meta.sub_loc.tolist() == [1792, 1536, 512]
    assert meta.main_plan["seq_lens"].tolist() == [256, 1024, 513]
    k_cpu, v_cpu = wl.pool.k_cache(0).cpu(), wl.pool.v_cache(0).cpu()
    out, lse = wl.op.forward_with_lse(wl.q, wl.k, wl.v, 0, wl.batch)
    rope = oracle_rope(wl.op, wl.theta)
    oplan = oracle_decode_plan(wl.group, wl.pending, wl.new_token_slots.cpu(), 16)
    k_rot = rope.rotate(wl.k.cpu().view(1, 2, 128), wl.batch.positions.cpu())
    O.store_kv(k_cpu.view(-1, 256), v_cpu.view(-1, 256), wl.new_token_slots.cpu(), k_rot.reshape(1, -1), wl.v.cpu())
    assert torch.equal(wl.pool.k_cache(0).cpu(), k_cpu) and torch.equal(wl.pool.v_cache(0).cpu(), v_cpu)
    eo, el, _ = O.forward_decode(oplan, wl.q.cpu().view(1, 8, 128), k_cpu, v_cpu, rope)
    assert_close(out, eo, torch.float32, "out")
    assert_close(lse, el, torch.float32, "lse")
    assert wl.alg_bytes > 1793 * 2048


@pytest.mark.parametrize("kernel", KERNELS)
@pytest.mark.parametrize("page", [1, 4, 16])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_cross_readers_duplicates_empty_blocks_and_implicit_self(kernel, page, dtype):
    op, cpu_pool, dev_pool, gen = make_op_and_pool(DEV, dtype, (8, 2, 64), page, 128, 1e4, seed=page, kernel=kernel)
    pages = Pages(page)
    common, left, right, empty = pages.block(page + 1, span=None), pages.block(page), pages.block(0), pages.block(0)
    other = pages.block(3 * page + 2)
    group = WorkerGroup(cache_structure=[[common, empty, right, left], [common, left, common], [other, common]],
                        write_to=[left, right, other])
    run_decode_parity(op, cpu_pool, dev_pool, group, pages, 1e4, gen)
    assert left.num_tokens == page and right.num_tokens == 0  # prepare/forward never commit growth


@pytest.mark.parametrize("kernel", KERNELS)
@pytest.mark.parametrize("heads,dim,rotary", [((16, 4, 256), 256, 256), ((16, 4, 256), 256, 64), ((8, 8, 128), 128, 128),
                                              ((16, 2, 256), 256, 256), ((4, 4, 64), 64, 32), ((32, 2, 128), 128, 64)])
def test_ragged_views_bf16(kernel, heads, dim, rotary):
    page = 16
    op, cpu_pool, dev_pool, gen = make_op_and_pool(DEV, torch.bfloat16, heads, page, 512, 1e7, rotary_dim=rotary,
                                                   seed=7, scale=1.0, kernel=kernel, max_pos=8192)
    pages = Pages(page)
    shared = pages.block(700)
    views, targets = [], []
    lengths = [[300], [17, 1000], [1, 2, 3], [640, 64], [255]]
    for ls in lengths:
        mine = [pages.block(n) for n in ls]
        views.append([shared] + mine)
        targets.append(mine[-1])
    run_decode_parity(op, cpu_pool, dev_pool, WorkerGroup(cache_structure=views, write_to=targets), pages, 1e7, gen,
                      scale=1.0)


@pytest.mark.parametrize("kernel", KERNELS)
def test_single_segment_fast_path_and_base2_lse(kernel):
    page = 16
    op, cpu_pool, dev_pool, gen = make_op_and_pool(DEV, torch.bfloat16, (8, 2, 128), page, 64, 1e4, kernel=kernel)
    pages = Pages(page)
    blocks = [pages.block(n) for n in (40, 16, 100)]
    group = WorkerGroup(cache_structure=[[b] for b in blocks])
    *_, meta = run_decode_parity(op, cpu_pool, dev_pool, group, pages, 1e4, gen, lse_base2=True)
    assert meta.max_segments == 1 and meta.n_aux == 0


@pytest.mark.parametrize("kernel", KERNELS)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_mrope_views_with_compressed_spans(kernel, dtype):
    """Interleaved mRoPE with blocks whose span differs from their token count
    (an image inside); decode queries are text, so rotations are scalar."""
    page = 16
    op, cpu_pool, dev_pool, gen = make_op_and_pool(DEV, dtype, (8, 2, 64), page, 128, 1e4, rotary_dim=32,
                                                   mrope_section=(8, 4, 4), seed=3, kernel=kernel)
    pages = Pages(page)
    common = pages.block(page + 1, span=1)
    a, b, c = pages.block(page), pages.block(page - 1, span=5), pages.block(0)
    group = WorkerGroup(cache_structure=[[common, a], [common, a, b], [common, b, a]], write_to=[a, b, c])
    run_decode_parity(op, cpu_pool, dev_pool, group, pages, 1e4, gen)


@pytest.mark.parametrize("kernel", KERNELS)
@pytest.mark.parametrize("heads,kv_heads,dim", [(16, 2, 256), (4, 4, 128)])
def test_zero_keys_unit_values_give_ones(kernel, heads, kv_heads, dim):
    page, workers = 16, 8
    k = torch.zeros(workers * 2, page, kv_heads, dim, device=DEV, dtype=torch.bfloat16)
    v = torch.ones_like(k)
    pool = SimpleNamespace(k_cache=lambda l: k, v_cache=lambda l: v)
    op = SharedCacheAttention(pool, torch.zeros(64, dim, device=DEV), heads, kv_heads, dim, page, torch.bfloat16, DEV,
                              kernel=kernel)
    for length in (31, 1, 16):
        blocks = []
        for w in range(workers):
            b = CacheBlock(DEV, page)
            b.page_starts = [2 * w * page, (2 * w + 1) * page][: -(-length // page)]
            b.num_tokens = length - 1  # the step appends the last token
            blocks.append(b)
        group = WorkerGroup(cache_structure=[[b] for b in blocks])
        pending = {id(b): None for b in blocks}
        slots = torch.tensor([b.page_starts[-1] + b.num_tokens % page for b in blocks], dtype=torch.int32, device=DEV)
        if any(not b.has_capacity for b in blocks):
            continue
        meta = op.prepare(group, pending, slots)
        batch = SimpleNamespace(attn_metadata=meta, positions=torch.zeros(workers, dtype=torch.int64, device=DEV),
                                out_loc=slots, mrope_positions=None)
        q = torch.randn(workers, heads * dim, device=DEV).bfloat16()
        out, lse = op.forward_with_lse(q, torch.zeros(workers, kv_heads * dim, device=DEV, dtype=torch.bfloat16),
                                       torch.ones(workers, kv_heads * dim, device=DEV, dtype=torch.bfloat16), 0, batch)
        assert torch.allclose(out.float(), torch.ones_like(out).float(), atol=2e-3)
        assert torch.allclose(lse, torch.full_like(lse, math.log(length)), atol=1e-4)


@pytest.mark.parametrize("kernel", KERNELS)
def test_scaled_batched_and_mrope_configurations(kernel):
    """Configurations 2 and 5 at reduced size through the workload builders."""
    for wl in (workloads.batched_decode(DEV, workers=6, shared_len=700, private_lo=20, private_hi=900, kernel=kernel),
               workloads.batched_decode(DEV, workers=5, shared_len=513, private_lo=1, private_hi=300, rotary_dim=64,
                                        kernel=kernel),
               workloads.mrope_decode(DEV, workers=3, blocks_per_view=3, block_len=400, image_tokens=64, kernel=kernel)):
        op = wl.op
        Hq, Hkv, D, P = op.num_qo_heads, op.num_kv_heads, op.head_dim, op.page_size
        k_cpu, v_cpu = wl.pool.k_cache(0).cpu(), wl.pool.v_cache(0).cpu()
        out, lse = op.forward_with_lse(wl.q, wl.k, wl.v, 0, wl.batch)
        rope = oracle_rope(op, wl.theta)
        oplan = oracle_decode_plan(wl.group, wl.pending, wl.new_token_slots.cpu(), P)
        assert wl.meta.sub_loc.tolist() == oplan.sub_loc
        W = wl.q.shape[0]
        k_rot = rope.rotate(wl.k.cpu().view(W, Hkv, D), wl.batch.positions.cpu())
        O.store_kv(k_cpu.view(-1, Hkv * D), v_cpu.view(-1, Hkv * D), wl.new_token_slots.cpu(), k_rot.reshape(W, -1),
                   wl.v.cpu())
        eo, el, _ = O.forward_decode(oplan, wl.q.cpu().view(W, Hq, D), k_cpu, v_cpu, rope)
        assert_close(out, eo, op.dtype, wl.name + " out")
        assert_close(lse, el, op.dtype, wl.name + " lse")
        assert wl.alg_bytes > 0 and wl.logical_bytes > 0


@pytest.mark.parametrize("heads,readers", [((16, 4, 256), 40), ((8, 8, 128), 70), ((16, 2, 64), 21)])
def test_many_readers_of_one_block_in_wide_tiles(heads, readers, monkeypatch):
    """Decode readers of one block through the wide matrix-core kernel (tiles of 128 or 256 MFMA rows, taken
    here on request; the planner takes them by itself only for blocks far too long for an oracle run), the
    private blocks and the leftover readers through the streaming kernel, all merged per row."""
    monkeypatch.setenv("VIEWATTN_PLAN", "wide_tile=%d" % (128 // (heads[0] // heads[1]) if heads[2] == 256 else
                                                           256 // (heads[0] // heads[1])))
    page = 16
    op, cpu_pool, dev_pool, gen = make_op_and_pool(DEV, torch.bfloat16, heads, page, 1400, 1e7, seed=11, scale=1.0,
                                                   kernel="auto", max_pos=8192)
    pages = Pages(page)
    shared = pages.block(1999)
    views, targets = [], []
    for w in range(readers):
        mine = pages.block(5 + 23 * (w % 9))
        views.append([shared, mine] if w % 5 else [mine, shared])
        targets.append(mine)
    *_, meta = run_decode_parity(op, cpu_pool, dev_pool, WorkerGroup(cache_structure=views, write_to=targets), pages,
                                 1e7, gen, scale=1.0)
    counts = meta.launch.counts
    assert counts.n_wide_items > 0 and counts.n_items > counts.n_wide_items


def test_forward_rejects_cpu_tensors_and_small_workspace():
    from async_llm_amd import native

    wl = workloads.batched_decode(DEV, workers=2, shared_len=600, private_lo=300, private_hi=400)
    with pytest.raises(native.ViewAttnError, match="GPU only"):
        wl.op.forward(wl.q.cpu(), wl.k, wl.v, 0, wl.batch)
    launch = wl.meta.launch
    if launch.counts.workspace_bytes:
        keep = launch.workspace
        launch.workspace = keep[:16]
        with pytest.raises(native.ViewAttnError, match="workspace needs"):
            wl.op.forward(wl.q, wl.k, wl.v, 0, wl.batch)
        launch.workspace = keep
