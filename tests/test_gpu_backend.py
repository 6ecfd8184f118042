"""The kernels behind the reference's regular backend interface
(attention/base.py:18-35): plain prefill, extend prefill over a cached prefix
and decode over token-slot tables, against the oracle's causal paged attention
(queries and keys arrive rotated, nothing is rotated here); recorded decode
batches replayed under new tables at two batch sizes (attention/fi.py:242-286)."""

from types import SimpleNamespace

import pytest
import torch

from async_llm_amd.attention_backend import ViewAttnBackend, ViewAttnMetadata, register
from async_llm_amd.kvcache import MHAKVCache
from oracle import view_attention_oracle as O
from tests.util import assert_close

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda")


def make_backend(dtype, heads, max_reqs=8, max_len=400, num_slots=4096, layers=2, seed=0):
    Hq, Hkv, D = heads
    pool = MHAKVCache(Hkv, layers, D, num_slots, 1, dtype, DEV)
    g = torch.Generator().manual_seed(seed)
    for l in range(layers):
        pool.k_cache(l).copy_((torch.randn(num_slots, 1, Hkv, D, generator=g) * D ** -0.5).to(dtype))
        pool.v_cache(l).copy_(torch.randn(num_slots, 1, Hkv, D, generator=g).to(dtype))
    # every request owns a scattered set of token slots
    perm = torch.randperm(num_slots, generator=g)[: max_reqs * max_len].to(torch.int32)
    page_table = perm.view(max_reqs, max_len).to(DEV)
    config = SimpleNamespace(num_qo_heads=Hq, num_kv_heads=Hkv, head_dim=D)
    return ViewAttnBackend(config, pool, page_table), pool, page_table, g


def make_batch(page_table, lens):
    """``lens``: (cached_len, extend_len) per request."""
    reqs = [SimpleNamespace(table_idx=i, cached_len=c, extend_len=e, device_len=c + e) for i, (c, e) in enumerate(lens)]
    out_loc = torch.cat([page_table[r.table_idx, r.cached_len: r.device_len] for r in reqs])
    decode = all(e == 1 for _, e in lens)
    return SimpleNamespace(reqs=reqs, padded_reqs=reqs, size=len(reqs), padded_size=len(reqs), out_loc=out_loc,
                           is_decode=decode, is_prefill=not decode, attn_metadata=None)


def expected(pool, page_table, batch, layer, q, k, v, heads):
    Hq, Hkv, D = heads
    k_cpu = pool.k_cache(layer).cpu().reshape(-1, Hkv, D).clone()
    v_cpu = pool.v_cache(layer).cpu().reshape(-1, Hkv, D).clone()
    loc = batch.out_loc.cpu().long()
    k_cpu[loc] = k.cpu().view(-1, Hkv, D)
    v_cpu[loc] = v.cpu().view(-1, Hkv, D)
    outs, row = [], 0
    for r in batch.padded_reqs:
        slots = page_table[r.table_idx, : r.device_len].cpu().long()
        qi = q.cpu().view(-1, Hq, D)[row: row + r.extend_len]
        o, _ = O.paged_attention(qi, k_cpu[slots], v_cpu[slots], causal=True)
        outs.append(o.reshape(r.extend_len, Hq * D))
        row += r.extend_len
    return torch.cat(outs), k_cpu, v_cpu


@pytest.mark.parametrize("dtype,heads", [(torch.bfloat16, (8, 2, 128)), (torch.float16, (4, 4, 64)),
                                         (torch.float32, (4, 2, 64))])
@pytest.mark.parametrize("lens", [
    [(0, 70), (0, 1), (0, 133)],            # plain prefill, no cached prefix
    [(64, 40), (17, 200), (300, 3)],        # extend prefill over cached prefixes
    [(99, 1), (0, 1), (257, 1), (31, 1)],   # decode
])
def test_backend_matches_causal_paged_attention(dtype, heads, lens):
    Hq, Hkv, D = heads
    backend, pool, page_table, g = make_backend(dtype, heads)
    batch = make_batch(page_table, lens)
    backend.prepare_metadata(batch)
    meta = batch.attn_metadata
    assert isinstance(meta, ViewAttnMetadata) and meta.page_size == 1
    n = sum(e for _, e in lens)
    assert meta.get_last_indices(len(lens)).tolist() == [sum(e for _, e in lens[: i + 1]) - 1 for i in range(len(lens))]
    q = (torch.randn(n, Hq * D, generator=g) * D ** -0.5).to(dtype).to(DEV)
    k = (torch.randn(n, Hkv * D, generator=g) * D ** -0.5).to(dtype).to(DEV)
    v = torch.randn(n, Hkv * D, generator=g).to(dtype).to(DEV)
    for layer in (0, 1):
        exp, k_cpu, v_cpu = expected(pool, page_table, batch, layer, q, k, v, heads)
        out = backend.forward(q, k, v, layer, batch)
        torch.cuda.synchronize()
        assert out.shape == (n, Hq * D) and out.dtype == dtype
        assert torch.equal(pool.k_cache(layer).cpu().reshape(-1, Hkv, D), k_cpu), "K rows are stored as given"
        assert torch.equal(pool.v_cache(layer).cpu().reshape(-1, Hkv, D), v_cpu)
        assert_close(out, exp, dtype, f"layer {layer}")


def test_recorded_decode_batches_follow_new_tables():
    dtype, heads = torch.bfloat16, (8, 2, 128)
    Hq, Hkv, D = heads
    backend, pool, page_table, g = make_backend(dtype, heads, max_reqs=8, max_len=400)
    backend.init_capture_graph(max_seq_len=400, bs_list=[2, 4])
    graphs, statics = {}, {}
    for bs in (4, 2):
        q_s = torch.zeros(bs, Hq * D, dtype=dtype, device=DEV)
        k_s = torch.zeros(bs, Hkv * D, dtype=dtype, device=DEV)
        v_s = torch.zeros(bs, Hkv * D, dtype=dtype, device=DEV)
        batch = make_batch(page_table, [(5 + i, 1) for i in range(bs)])
        loc_s = batch.out_loc.clone()
        batch.out_loc = loc_s
        backend.prepare_for_capture(batch)
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            backend.forward(q_s, k_s, v_s, 0, batch)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            out_s = backend.forward(q_s, k_s, v_s, 0, batch)
        graphs[bs], statics[bs] = graph, (q_s, k_s, v_s, loc_s, out_s)
    for bs, lens in ((4, [(120, 1), (7, 1), (399, 1), (64, 1)]), (2, [(250, 1), (33, 1)]),
                     (4, [(1, 1), (300, 1), (15, 1), (16, 1)]), (2, [(0, 1), (398, 1)])):
        q_s, k_s, v_s, loc_s, out_s = statics[bs]
        batch = make_batch(page_table, lens)
        backend.prepare_metadata(batch)  # the scheduler plans every batch; replay then moves it to the fixed tables
        backend.prepare_for_replay(batch)
        q = (torch.randn(bs, Hq * D, generator=g) * D ** -0.5).to(dtype).to(DEV)
        k = (torch.randn(bs, Hkv * D, generator=g) * D ** -0.5).to(dtype).to(DEV)
        v = torch.randn(bs, Hkv * D, generator=g).to(dtype).to(DEV)
        exp, k_cpu, v_cpu = expected(pool, page_table, batch, 0, q, k, v, heads)
        q_s.copy_(q); k_s.copy_(k); v_s.copy_(v); loc_s.copy_(batch.out_loc)
        for _ in range(2):  # a second replay of the same tables gives the same rows
            graphs[bs].replay()
            torch.cuda.synchronize()
            assert_close(out_s, exp, dtype, f"bs {bs}, lens {lens}")
        assert torch.equal(pool.k_cache(0).cpu().reshape(-1, Hkv, D), k_cpu)


def test_registration_and_rejected_batches():
    class Registry(dict):
        def register(self, name):
            def add(fn):
                self[name] = fn
                return fn
            return add

    registry = Registry()
    register(registry)
    backend, pool, page_table, g = make_backend(torch.bfloat16, (8, 2, 128))
    made = registry["viewattn"](backend.config, kv_cache=pool, page_table=page_table)
    assert isinstance(made, ViewAttnBackend)
    bad = make_batch(page_table, [(0, 4)])
    bad.padded_reqs[0].device_len = 2
    with pytest.raises(ValueError, match="extends by 4"):
        backend.prepare_metadata(bad)
    backend.init_capture_graph(max_seq_len=50, bs_list=[2])
    batch = make_batch(page_table, [(3, 1), (60, 1)])
    with pytest.raises(ValueError, match="longer than the recorded maximum"):
        backend.prepare_for_capture(batch)
