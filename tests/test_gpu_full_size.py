"""Properties of the product path at the FULL sizes of the benchmark
configurations, where an element-wise oracle run is too slow for a test:

* zero keys and unit values (the reference's only absolute known answer,
  tests/core/test_attention_workspace.py:121-125): every score is 0, so the output
  is exactly 1 and the LSE of a row is the log of the NUMBER OF TOKENS IT SEES --
  which checks, per row and at full scale, that every visible token of every
  segment is covered exactly once (chunks, shared tiles, causal diagonal, merge);
* the result does not depend on how the planner cuts the work (another chunk size
  and tile shape give the same output);
* attention is linear in V: doubling every value (exact in bf16) doubles the output
  bit for bit and leaves the LSE alone.
"""

import os

import pytest
import torch

from async_llm_amd import native, workloads

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda")


def _zero_keys_unit_values(wl):
    for layer in range(1):
        wl.pool.k_cache(layer).zero_()
        wl.pool.v_cache(layer).fill_(1.0)
    k0 = torch.zeros_like(wl.k)
    v1 = torch.ones_like(wl.v)
    return wl.op.forward_with_lse(wl.q, k0, v1, 0, wl.batch)


def test_batched_decode_full_size_counts_every_token_once():
    wl = workloads.batched_decode(DEV, layers=1)  # configuration 2: 64 requests, ~550 k distinct tokens
    out, lse = _zero_keys_unit_values(wl)
    assert torch.equal(out, torch.ones_like(out))
    tokens = torch.tensor([sum(b.num_tokens for b in view) + 1 for view in wl.group.cache_structure], dtype=torch.float64)
    want = tokens.log()[:, None].expand(-1, wl.op.num_qo_heads)
    assert torch.allclose(lse.double().cpu(), want, atol=1e-5, rtol=0), (lse.double().cpu() - want).abs().max()


def test_long_shared_block_goes_wide_by_itself_and_counts_every_token_once():
    # 64 readers of a 32768-token block: narrow tiles would stream it 16 times, the planner cuts the readers
    # into two wide tiles (a launch of their own) without being asked
    wl = workloads.batched_decode(DEV, layers=1, shared_len=32768)
    assert wl.meta.launch.counts.n_wide_items > 0
    out, lse = _zero_keys_unit_values(wl)
    assert torch.equal(out, torch.ones_like(out))
    tokens = torch.tensor([sum(b.num_tokens for b in view) + 1 for view in wl.group.cache_structure], dtype=torch.float64)
    want = tokens.log()[:, None].expand(-1, wl.op.num_qo_heads)
    assert torch.allclose(lse.double().cpu(), want, atol=1e-5, rtol=0), (lse.double().cpu() - want).abs().max()


def test_view_prefill_full_size_counts_every_visible_token_once():
    wl = workloads.view_prefill(DEV, layers=1)  # configuration 3: 8 x 2048 new tokens over ~42 k tokens of view each
    out, lse = _zero_keys_unit_values(wl)
    assert torch.equal(out, torch.ones_like(out))
    want = []
    for s in wl.specs:
        before = sum(b.num_tokens for b in s.context) + s.self_prefix_len
        want.append(torch.arange(1, s.num_new + 1, dtype=torch.float64) + before)
    want = torch.cat(want).log()[:, None].expand(-1, wl.op.num_qo_heads)
    assert torch.allclose(lse.double().cpu(), want, atol=1e-5, rtol=0), (lse.double().cpu() - want).abs().max()


def test_mixed_batch_full_size_counts_every_visible_token_once():
    wl = workloads.mixed_batch(DEV, layers=1)  # configuration 4: 48 decode rows + 4 chunks of 512 in one launch
    out, lse = _zero_keys_unit_values(wl)
    assert torch.equal(out, torch.ones_like(out))
    # decode rows see their whole view plus this step's token; row u of a chunk sees its context, the
    # prefix of its own block and new tokens 0..u
    want = [torch.tensor([sum(b.num_tokens for b in view) + 1 for view in wl.group.cache_structure],
                         dtype=torch.float64)]
    for s in wl.specs:
        before = sum(b.num_tokens for b in s.context) + s.self_prefix_len
        want.append(torch.arange(1, s.num_new + 1, dtype=torch.float64) + before)
    want = torch.cat(want).log()[:, None].expand(-1, wl.op.num_qo_heads)
    assert lse.shape == want.shape
    assert torch.allclose(lse.double().cpu(), want, atol=1e-5, rtol=0), (lse.double().cpu() - want).abs().max()


def test_mrope_decode_full_size_counts_every_token_once():
    # configuration 5: 8 requests x 8 blocks x 16384 tokens; the only configuration whose pool byte
    # offsets pass 2^31 (65 k pages of 32 KB per layer)
    wl = workloads.mrope_decode(DEV, layers=1)
    assert wl.pool.k_cache(0).numel() * wl.pool.k_cache(0).element_size() > 2 ** 31
    out, lse = _zero_keys_unit_values(wl)
    assert torch.equal(out, torch.ones_like(out))
    tokens = torch.tensor([sum(b.num_tokens for b in view) + 1 for view in wl.group.cache_structure], dtype=torch.float64)
    assert tokens.min() == 8 * 16384 + 1
    want = tokens.log()[:, None].expand(-1, wl.op.num_qo_heads)
    assert torch.allclose(lse.double().cpu(), want, atol=1e-5, rtol=0), (lse.double().cpu() - want).abs().max()


def test_mrope_decode_full_size_reads_the_right_rows():
    # zero keys make every row of V weigh the same, so the output is the mean of the value rows the
    # view's page tables name.  Every value row holds the number of the 128 MB region of the pool it
    # lives in (exact in bf16), so rows fetched through an offset folded to 32 bits (the pool is 4 GB
    # per layer) come from other regions and move the mean.
    wl = workloads.mrope_decode(DEV, layers=1)
    k_pool, v_pool = wl.pool.k_cache(0), wl.pool.v_cache(0)
    k_pool.zero_()
    slots = torch.arange(v_pool.shape[0] * v_pool.shape[1], device=DEV)
    tag = slots >> 16  # 65536 slots of 2 KB: region number, 0..16
    v_pool.view(slots.numel(), -1).copy_(tag[:, None].to(v_pool.dtype).expand(-1, v_pool.shape[2] * v_pool.shape[3]))
    v_new = torch.zeros_like(wl.v)
    out, _ = wl.op.forward_with_lse(wl.q, torch.zeros_like(wl.k), v_new, 0, wl.batch)
    P = wl.op.page_size
    want = []
    for w, view in enumerate(wl.group.cache_structure):
        starts = torch.tensor([s for b in view for s in b.page_starts], dtype=torch.int64)
        rows = (starts[:, None] + torch.arange(P)[None, :]).reshape(-1)
        n = sum(b.num_tokens for b in view)
        assert rows.numel() == n  # full pages; the appended token (value 0) lives in a pending page
        want.append(tag.cpu()[rows].double().sum() / (n + 1))
    want = torch.stack(want)[:, None].expand(-1, out.shape[1])
    assert torch.allclose(out.double().cpu(), want, atol=0.0, rtol=6e-3), (out.double().cpu() - want).abs().max()


@pytest.mark.parametrize("name", ["batched_decode", "view_prefill"])
def test_full_size_result_is_independent_of_the_work_decomposition(name):
    build = getattr(workloads, name)
    wl = build(DEV, layers=1)
    out, lse = wl.op.forward_with_lse(wl.q, wl.k, wl.v, 0, wl.batch)
    os.environ["VIEWATTN_PLAN"] = "kv_chunk=704,wide_tile=16" if name == "view_prefill" else "kv_chunk=448,q_tile=2"
    try:
        other = build(DEV, layers=1)  # same seed: same inputs, another plan
    finally:
        del os.environ["VIEWATTN_PLAN"]
    assert other.meta.launch.counts.n_items != wl.meta.launch.counts.n_items
    out2, lse2 = other.op.forward_with_lse(other.q, other.k, other.v, 0, other.batch)
    assert torch.allclose(out2.float(), out.float(), atol=2e-2, rtol=1e-2)
    assert torch.allclose(lse2, lse, atol=2e-3, rtol=1e-3)


def test_batched_decode_full_size_is_linear_in_values():
    wl = workloads.batched_decode(DEV, layers=1)
    out, lse = wl.op.forward_with_lse(wl.q, wl.k, wl.v, 0, wl.batch)
    wl.pool.v_cache(0).mul_(2.0)
    out2, lse2 = wl.op.forward_with_lse(wl.q, wl.k, wl.v * 2, 0, wl.batch)
    assert torch.equal(out2, out * 2) and torch.equal(lse2, lse)


@pytest.mark.parametrize("name", ["view_prefill", "mixed_batch", "batched_decode"])
def test_full_size_results_repeat_bit_for_bit(name):
    """No atomics and a fixed merge order: one plan gives the same bits every time.  A tile read from a ring
    buffer before it has landed, or after it was refilled, would show up here as a run that differs."""
    wl = getattr(workloads, name)(DEV, layers=1)
    first = None
    for _ in range(5):
        out, lse = wl.op.attend(wl.q, 0, wl.meta, return_lse=True)
        torch.cuda.synchronize()
        if first is None:
            first = (out.clone(), lse.clone())
            assert torch.isfinite(out.float()).all() and torch.isfinite(lse).all()
        else:
            assert torch.equal(out, first[0]) and torch.equal(lse, first[1])
