"""Recorded launches replayed under changing plans: ``forward`` is captured
once into a HIP graph at the buffers' capacity, then every replay follows a new
``plan`` written into the same device tables, and is checked against the CPU
oracle and against the unrecorded (packed-plan) product path.  Scenario of the
reference's tests/core/test_shared_decode_attention_graph.py:16-107 (replays
for 2, 4, 1, 3, 4 active workers of 4; rows of inactive workers come back zero)
and tests/core/test_shared_prefill_attention_graph.py:14-135 (ragged batches
replayed through one graph)."""

from types import SimpleNamespace

import pytest
import torch

from async_llm_amd.shared_cache import CacheBlock, WorkerGroup
from async_llm_amd.shared_cache.attention_graph import SharedDecodeAttentionBuffers, SharedPrefillAttentionBuffers
from async_llm_amd.shared_cache.session_planning import plan_decode_writes
from oracle import view_attention_oracle as O
from tests.test_gpu_prefill import common_blocks, make_specs
from tests.util import (assert_close, make_op_and_pool, oracle_decode_plan, oracle_prefill, oracle_rope,
                        prefill_inputs)

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda")


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


def record(op, statics, meta):
    """Warm the launches up on a side stream, then capture one forward."""
    q, k, v, positions, out_loc, mrope_positions = statics
    batch = SimpleNamespace(attn_metadata=meta, positions=positions, out_loc=out_loc, mrope_positions=mrope_positions)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        op.forward_with_lse(q, k, v, 0, batch)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out, lse = op.forward_with_lse(q, k, v, 0, batch)
    return graph, out, lse


@pytest.mark.parametrize("page,dtype,rotary", [(16, torch.bfloat16, 64), (4, torch.float32, 32)])
def test_decode_graph_follows_each_new_plan(page, dtype, rotary):
    W, depth, theta = 4, 3, 1e4
    Hq, Hkv, D = 8, 2, 64
    op, cpu_pool, dev_pool, gen = make_op_and_pool(DEV, dtype, (Hq, Hkv, D), page, 512, theta, rotary_dim=rotary,
                                                   seed=11, max_pos=2048)
    buffers = SharedDecodeAttentionBuffers(op, W, depth, max_pages=256, dummy_slots=torch.zeros(W, dtype=torch.int64))
    op.prepare_workspace([buffers])
    workspace = op._workspace.data_ptr()
    q_s = torch.zeros(W, Hq * D, dtype=dtype, device=DEV)
    k_s = torch.zeros(W, Hkv * D, dtype=dtype, device=DEV)
    v_s = torch.zeros(W, Hkv * D, dtype=dtype, device=DEV)
    pos_s = torch.zeros(W, dtype=torch.int64, device=DEV)
    loc_s = torch.full((W,), -1, dtype=torch.int32, device=DEV)
    graph, out_s, lse_s = record(op, (q_s, k_s, v_s, pos_s, loc_s, None), buffers.meta)
    pool_before = [t.clone() for t in dev_pool]
    graph.replay()  # the all-empty plan: nothing stored, zero rows
    torch.cuda.synchronize()
    assert not out_s.any() and torch.isinf(lse_s).all()
    assert all(torch.equal(a, b) for a, b in zip(pool_before, dev_pool))

    pages = Pages(page, first=1)
    prompt = pages.block(70)
    rope = oracle_rope(op, theta)
    for step, n in enumerate((2, 4, 1, 3, 4)):
        own = [pages.block(5 + 13 * ((step + w) % 4)) for w in range(n)]
        side_block = pages.block(page * 2)  # full: its writer opens a page
        views, targets = [], []
        for w in range(n):
            view = [prompt, own[(w + 1) % n], own[w]] if w % 2 == 0 else [own[w], prompt]
            views.append(view[:depth])
            targets.append(own[w])
        if n >= 3:  # one worker writes a block outside its view
            views[n - 1] = [prompt]
            targets[n - 1] = side_block
        group = WorkerGroup(cache_structure=views, write_to=targets)
        pending, slots, write_pos = plan_decode_writes(group, page, pages, DEV)
        meta = op.prepare(group, pending, slots, graph_buffers=buffers)
        assert meta is buffers.meta and op._workspace.data_ptr() == workspace
        q = (torch.randn(n, Hq * D, generator=gen) * D ** -0.5).to(dtype)
        k = (torch.randn(n, Hkv * D, generator=gen) * D ** -0.5).to(dtype)
        v = (torch.randn(n, Hkv * D, generator=gen) * D ** -0.5).to(dtype)
        positions = torch.tensor(write_pos, dtype=torch.int64)
        q_s.zero_(); k_s.zero_(); v_s.zero_(); pos_s.zero_(); loc_s.fill_(-1)
        q_s[:n], k_s[:n], v_s[:n] = q.to(DEV), k.to(DEV), v.to(DEV)
        pos_s[:n], loc_s[:n] = positions.to(DEV), slots
        graph.replay()
        torch.cuda.synchronize()
        out, lse = out_s.clone(), lse_s.clone()

        k_cpu, v_cpu = cpu_pool
        k_rot = rope.rotate(k.view(n, Hkv, D), positions)
        O.store_kv(k_cpu.view(-1, Hkv * D), v_cpu.view(-1, Hkv * D), slots.cpu(), k_rot.reshape(n, -1), v)
        assert torch.equal(dev_pool[0].cpu(), k_cpu) and torch.equal(dev_pool[1].cpu(), v_cpu), f"pool, step {step}"
        oplan = oracle_decode_plan(group, pending, slots.cpu(), page)
        exp_out, exp_lse, _ = O.forward_decode(oplan, q.view(n, Hq, D), k_cpu, v_cpu, rope)
        assert_close(out[:n], exp_out, dtype, f"out, step {step}")
        assert_close(lse[:n], exp_lse, dtype, f"lse, step {step}")
        assert not out[n:].any() and torch.isinf(lse[n:]).all(), f"inactive rows, step {step}"

        # the unrecorded path over the packed plan of the same step agrees
        plain = op.prepare(group, pending, slots)
        batch = SimpleNamespace(attn_metadata=plain, positions=positions.to(DEV), out_loc=slots, mrope_positions=None)
        eager_out, eager_lse = op.forward_with_lse(q.to(DEV), k.to(DEV), v.to(DEV), 0, batch)
        assert_close(out[:n], eager_out.float(), dtype, f"recorded vs unrecorded out, step {step}")
        assert_close(lse[:n], eager_lse, dtype, f"recorded vs unrecorded lse, step {step}")

        # a second replay of the same plan reproduces the first bit for bit
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out_s, out) and torch.equal(lse_s, lse), f"second replay, step {step}"


@pytest.mark.parametrize("mrope", [False, True])
def test_prefill_graph_follows_each_new_batch(mrope):
    page, heads, dtype, theta = 16, (4, 2, 64), torch.bfloat16, 1e4
    Hq, Hkv, D = heads
    workers, depth, rows = 4, 3, 320
    op, cpu_pool, dev_pool, gen = make_op_and_pool(
        DEV, dtype, heads, page, 64, theta, rotary_dim=32 if mrope else 64,
        mrope_section=(8, 4, 4) if mrope else None, seed=735, scale=1.0, max_pos=2048)
    buffers = SharedPrefillAttentionBuffers(op, workers, depth, rows, max_pages=128)
    op.prepare_workspace([buffers])
    assert buffers.capacity.max_wide_items > 0  # the capacity covers both launches
    q_s = torch.zeros(rows, Hq * D, dtype=dtype, device=DEV)
    k_s = torch.zeros(rows, Hkv * D, dtype=dtype, device=DEV)
    v_s = torch.zeros(rows, Hkv * D, dtype=dtype, device=DEV)
    pos_s = torch.zeros(rows, dtype=torch.int64, device=DEV)
    mpos_s = torch.zeros(3, rows, dtype=torch.int64, device=DEV) if mrope else None
    loc_s = torch.full((rows,), -1, dtype=torch.int32, device=DEV)
    graph, out_s, lse_s = record(op, (q_s, k_s, v_s, pos_s, loc_s, mpos_s), buffers.meta)

    common = common_blocks(page, mrope)
    for turn, lengths in ((0, [1]), (2, [63, 65, 3]), (3, [138, 91, 1]), (4, [64] * 4), (5, [9, 7])):
        specs = make_specs(common, lengths, turn, page, mrope, full_context=(turn == 4))
        meta = op.prepare_prefill_batch(specs, graph_buffers=buffers)
        assert meta is buffers.meta
        positions, mrope_positions, out_loc, q, k, v = prefill_inputs(op, specs, gen, scale=1.0)
        n = q.shape[0]
        q_s.zero_(); k_s.zero_(); v_s.zero_(); pos_s.zero_(); loc_s.fill_(-1)
        q_s[:n], k_s[:n], v_s[:n] = q.to(DEV), k.to(DEV), v.to(DEV)
        pos_s[:n], loc_s[:n] = positions.to(DEV), out_loc.to(DEV)
        if mrope:
            mpos_s.zero_()
            mpos_s[:, :n] = mrope_positions.to(DEV)
        graph.replay()
        torch.cuda.synchronize()
        out, lse = out_s.clone(), lse_s.clone()
        exp_out, exp_lse = oracle_prefill(op, cpu_pool, specs, theta, positions, mrope_positions, out_loc, q, k, v)
        assert torch.equal(dev_pool[1].cpu(), cpu_pool[1]), f"V pool, turn {turn}"
        assert_close(out[:n], exp_out, dtype, f"out, turn {turn}")
        assert_close(lse[:n], exp_lse, dtype, f"lse, turn {turn}")
        assert not out[n:].any() and torch.isinf(lse[n:]).all(), f"unused rows, turn {turn}"
        assert meta.get_last_indices(len(specs))[:len(specs)].tolist() == \
            [sum(lengths[:i + 1]) - 1 for i in range(len(lengths))]
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out_s, out) and torch.equal(lse_s, lse), f"second replay, turn {turn}"
