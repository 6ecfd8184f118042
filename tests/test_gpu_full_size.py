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

import math
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
    assert torch.isfinite(lse).all() and (lse > math.log(512)).all()  # every row sees at least the shared prompt


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
