"""Pins the CPU oracle before anything is compared with it.

Rotation: closed-form HF neox RoPE with the reference's per-dtype tolerances
(tests/core/test_rope_correction_kernel.py:49-170, test_shared_cache.py:178-258).
mRoPE: reductions to 1-D RoPE, brute-forced section rule, fixtures.
Attention/merge: fp64 brute force, torch SDPA, the concatenated-view invariant,
and the K=0/V=1 known answer (tests/core/test_attention_workspace.py:121-125).
"""

import json
import math
import os

import pytest
import torch
import torch.nn.functional as F

from oracle import view_attention_oracle as O

HERE = os.path.dirname(os.path.abspath(__file__))


def hf_rope(x, positions, base=10000.0, rotary_dim=None):
    """HF-style neox RoPE from its definition, fp32."""
    rd = x.shape[-1] if rotary_dim is None else rotary_dim
    half = rd // 2
    inv = 1.0 / (base ** (torch.arange(0, rd, 2, dtype=torch.float) / rd))
    ang = positions.float().unsqueeze(-1) * inv.unsqueeze(0)
    c, s = ang.cos().unsqueeze(1), ang.sin().unsqueeze(1)
    a, b = x.float()[..., :half], x.float()[..., half:rd]
    return torch.cat([c * a - s * b, c * b + s * a, x.float()[..., rd:]], dim=-1)


@pytest.mark.parametrize("dtype,atol", [(torch.float32, 1e-5), (torch.float16, 5e-3), (torch.bfloat16, 3e-2)])
def test_rope_correction_dtype_matrix(dtype, atol):
    torch.manual_seed(0)
    keys = torch.randn(8, 4, 64, dtype=dtype)
    corr = torch.tensor([0, 5, -3, 17, -12, 42, 99, -50])
    cs = O.build_cos_sin_cache(64, 256, 10000.0)
    got = O.apply_rope_correction(keys, corr, cs)
    assert got.dtype == dtype and got.shape == keys.shape
    assert torch.allclose(got.float(), hf_rope(keys, corr).to(dtype).float(), atol=atol)


def test_rope_correction_identity_boundary_negative_empty_roundtrip():
    torch.manual_seed(1)
    cs = O.build_cos_sin_cache(64, 128, 10000.0)
    keys = torch.randn(5, 2, 64)
    assert torch.allclose(O.apply_rope_correction(keys, torch.zeros(5, dtype=torch.int64), cs), keys, atol=1e-6)
    edge = torch.tensor([127, -127, -100, -1, 64])
    assert torch.allclose(O.apply_rope_correction(keys, edge, cs), hf_rope(keys, edge), atol=1e-5)
    # offsets beyond the table are clamped to its last row
    far = torch.tensor([500, -500, 127, -127, 0])
    assert torch.equal(O.apply_rope_correction(keys, far, cs),
                       O.apply_rope_correction(keys, torch.tensor([127, -127, 127, -127, 0]), cs))
    out = O.apply_rope_correction(torch.zeros(0, 2, 64), torch.zeros(0, dtype=torch.int64), cs)
    assert out.shape == (0, 2, 64)
    fwd = O.apply_rope_correction(keys, torch.full((5,), 23), cs)
    back = O.apply_rope_correction(fwd, torch.full((5,), -23), cs)
    assert torch.allclose(back, keys, atol=1e-5)


def test_rope_partial_passes_tail_through():
    torch.manual_seed(2)
    x = torch.randn(6, 3, 64)
    pos = torch.tensor([0, 1, 7, 30, -4, 100])
    cs = O.build_cos_sin_cache(16, 128, 1e6)
    got = O.rope_partial(x, pos, cs, 16)
    assert torch.equal(got[..., 16:], x[..., 16:])
    assert torch.allclose(got, hf_rope(x, pos, 1e6, 16), atol=1e-5)


@pytest.mark.parametrize("section,rd", [((8, 4, 4), 32), ((24, 20, 20), 128)])
def test_mrope_reductions_and_section_rule(section, rd):
    torch.manual_seed(3)
    D, base = rd * 2, 1e4
    x = torch.randn(7, 2, D)
    inv = O.mrope_inv_freq(rd, base)
    pos = torch.tensor([0, 1, 5, 17, 100, 1000, 12352])
    # a scalar position (same on all three axes) is plain partial 1-D RoPE
    got = O.rope_mrope(x, pos, inv, section, rd)
    assert torch.allclose(got, hf_rope(x, pos, base, rd), atol=2e-4)
    assert torch.equal(got[..., rd:], x[..., rd:])
    assert torch.equal(O.rope_mrope(x, pos.expand(3, -1), inv, section, rd), got)
    # genuine 3-D positions: brute force per rotary pair with the interleave rule
    pos3 = torch.stack([pos, pos * 2 + 1, pos + 3])
    got3 = O.rope_mrope(x, pos3, inv, section, rd)
    half = rd // 2
    want = x.clone()
    for i in range(half):
        axis = 0
        if i % 3 == 1 and i < 3 * section[1]:
            axis = 1
        if i % 3 == 2 and i < 3 * section[2]:
            axis = 2
        ang = pos3[axis].float() * inv[i]
        c, s = ang.cos()[:, None], ang.sin()[:, None]
        want[..., i] = x[..., i] * c - x[..., i + half] * s
        want[..., i + half] = x[..., i + half] * c + x[..., i] * s
    assert torch.allclose(got3, want, atol=1e-5)
    # the axes really are used: temporal pairs ignore h/w, and vice versa
    n_h = len([i for i in range(half) if i % 3 == 1 and i < 3 * section[1]])
    n_w = len([i for i in range(half) if i % 3 == 2 and i < 3 * section[2]])
    assert (n_h, n_w, half - n_h - n_w) == (section[1], section[2], section[0])


def test_mrope_low_precision_rounds_like_torch():
    torch.manual_seed(4)
    x = torch.randn(4, 2, 64).bfloat16()
    pos = torch.tensor([3, 9, 27, 81])
    inv = O.mrope_inv_freq(32, 1e4)
    got = O.rope_mrope(x, pos, inv, (8, 4, 4), 32)
    assert got.dtype == torch.bfloat16
    assert torch.allclose(got.float(), hf_rope(x, pos, 1e4, 32), atol=3e-2)


def test_get_rope_index_known_answers_and_fixtures():
    pos = O.get_rope_index([0] * 5, 2)
    assert torch.equal(pos, torch.arange(5).view(1, -1).expand(3, -1))
    pos = O.get_rope_index([0, 0, 1, 1, 1, 1, 0, 0, 0], 2, [[1, 4, 4]])
    assert pos[0].tolist() == [0, 1, 2, 2, 2, 2, 4, 5, 6]
    assert pos[1].tolist() == [0, 1, 2, 2, 3, 3, 4, 5, 6]
    assert pos[2].tolist() == [0, 1, 2, 3, 2, 3, 4, 5, 6]
    with open(os.path.join(HERE, "golden", "mrope_positions.json")) as f:
        for case in json.load(f):
            got = O.get_rope_index(case["mm_token_type_ids"], case["spatial_merge_size"], case["image_grid_thw"])
            assert got.tolist() == case["rope_positions"], case["source"]


def test_oracle_block_arithmetic():
    b = O.OBlock(4)
    assert (b.num_pages, b.last_page_len, b.has_capacity, b.pages_needed(9)) == (0, 0, False, 3)
    b.grow_pages([0, 4], 5)
    assert (b.last_page_len, b.free_tail, b.pages_needed(3), b.pages_needed(4), b.pages_needed(12)) == (1, 3, 0, 1, 3)
    for _ in range(3):
        b.append_token(None)
    b.append_token(8)
    assert b.page_starts == [0, 4, 8] and b.token_slots() == list(range(9))


def test_oracle_decode_plan_known_answer():
    for P in (1, 4, 16):
        common, left = O.OBlock(P, [7 * P, 2 * P], P + 1, 1), O.OBlock(P, [11 * P], P)
        right, empty = O.OBlock(P), O.OBlock(P)
        plan = O.plan_decode([[common, empty, right, left], [common, left, common]], [left, right],
                             {id(left): 13 * P, id(right): 17 * P}, [13 * P, 17 * P], P)
        pages = [plan.kv_indices[a:b] for a, b in zip(plan.kv_indptr, plan.kv_indptr[1:])]
        assert pages == [[7, 2], [17], [11, 13], [7, 2], [11, 13], [7, 2]]
        assert plan.seq_lens == [P + 1, 1, P + 1, P + 1, P + 1, P + 1]
        assert plan.sub_loc == [P + 2, P + 1, P, P + 2, P + 1, 0, 0]
        assert plan.aux_slots == [17 * P]
        assert left.page_starts == [11 * P] and right.page_starts == []


def test_oracle_decode_writes_known_answer():
    a, b, c = O.OBlock(4, [12], 4), O.OBlock(4, [32], 2), O.OBlock(4)
    calls = []

    def alloc(n):
        calls.append(n)
        return [40, 52]

    pending, slots, pos = O.plan_decode_writes([a, b, c], 4, alloc)
    assert calls == [2] and pending == {id(a): 40, id(b): None, id(c): 52}
    assert slots == [40, 34, 52] and pos == [4, 2, 0]


def test_oracle_prefill_plan_worked_example():
    shared = O.OBlock(4, [28, 8], 5, 2)
    plan = O.plan_prefill_batch([O.OPrefillSpec([shared, shared], [80, 84], 3, 2, 1,
                                                torch.arange(3).expand(3, -1))], 4)
    assert plan.sub_loc[0].tolist() == [5, 6, 7, 3, 4, 5, 1, 2, 3]
    assert plan.ctx["kv_indices"] == [7, 2, 7, 2] and plan.ctx["seq_lens"] == [5, 5] and plan.ctx["last_page_len"] == [1, 1]
    assert plan.own["kv_indices"] == [20, 21] and plan.own["seq_lens"] == [5] and plan.own["last_page_len"] == [1]
    assert plan.max_segments == 3 and plan.last_indices == [2]


# ---------------------------------------------------------------------------
# attention arithmetic
# ---------------------------------------------------------------------------
def brute_attention(q, keys, values, causal):
    """Per (row, head) loops in fp64, straight from the definition."""
    n, Hq, D = q.shape
    L, Hkv, _ = keys.shape
    g = Hq // Hkv
    out = torch.zeros(n, Hq, D, dtype=torch.float64)
    lse = torch.zeros(n, Hq, dtype=torch.float64)
    for i in range(n):
        limit = L - n + i if causal else L - 1
        for h in range(Hq):
            s = [float(q[i, h].double() @ keys[t, h // g].double()) / math.sqrt(D) for t in range(limit + 1)]
            top = max(s)
            z = sum(math.exp(v - top) for v in s)
            lse[i, h] = top + math.log(z)
            for t, v in enumerate(s):
                out[i, h] += math.exp(v - top) / z * values[t, h // g].double()
    return out, lse


@pytest.mark.parametrize("causal", [False, True])
def test_paged_attention_brute_force_and_sdpa(causal):
    torch.manual_seed(5)
    q, k, v = torch.randn(3, 4, 16), torch.randn(7, 2, 16), torch.randn(7, 2, 16)
    out, lse = O.paged_attention(q, k, v, causal=causal, math_dtype=torch.float64, out_dtype=torch.float64)
    bo, bl = brute_attention(q, k, v, causal)
    assert torch.allclose(out, bo, atol=1e-12) and torch.allclose(lse, bl, atol=1e-12)
    if not causal:
        want = F.scaled_dot_product_attention(q.double().transpose(0, 1)[None], k.double().transpose(0, 1)[None],
                                              v.double().transpose(0, 1)[None], enable_gqa=True)[0].transpose(0, 1)
        assert torch.allclose(out, want, atol=1e-12)


def test_gather_tokens_follows_page_table():
    paged = torch.arange(6 * 4 * 1 * 2, dtype=torch.float32).view(6, 4, 1, 2)
    got = O.gather_tokens(paged, [5, 0, 3], 9)
    want = torch.cat([paged[5], paged[0], paged[3][:1]])
    assert torch.equal(got, want)


def test_merge_states_equals_joint_softmax_and_padding_is_weightless():
    torch.manual_seed(6)
    q = torch.randn(2, 4, 8)
    ks = [torch.randn(n, 2, 8) for n in (3, 5, 1)]
    vs = [torch.randn(n, 2, 8) for n in (3, 5, 1)]
    parts = [O.paged_attention(q, k, v, math_dtype=torch.float64, out_dtype=torch.float64) for k, v in zip(ks, vs)]
    v_pad = torch.stack([p[0] for p in parts] + [torch.zeros(2, 4, 8, dtype=torch.float64)], dim=1)
    s_pad = torch.stack([p[1] for p in parts] + [torch.full((2, 4), O.PAD_LSE, dtype=torch.float64)], dim=1)
    merged, lse = O.merge_states(v_pad, s_pad)
    want, wlse = O.paged_attention(q, torch.cat(ks), torch.cat(vs), math_dtype=torch.float64, out_dtype=torch.float64)
    assert torch.allclose(merged, want, atol=1e-12) and torch.allclose(lse, wlse, atol=1e-12)
    # an all-padding row stays finite
    m2, l2 = O.merge_states(torch.zeros(1, 2, 4, 8), torch.full((1, 2, 4), O.PAD_LSE))
    assert torch.isfinite(m2).all() and torch.isfinite(l2).all() and m2.abs().max() == 0


def _random_view_case(seed, P, aux, dup):
    """Blocks with UNROTATED keys kept aside so the concatenated-view closed form
    can be evaluated; returns everything the two evaluations need."""
    g = torch.Generator().manual_seed(seed)
    Hq, Hkv, D, base = 4, 2, 16, 1e4
    lens = [5, 0, 2 * P + 1, 3]
    raw_k = [torch.randn(n + 1, Hkv, D, generator=g, dtype=torch.float64) for n in lens]
    val = [torch.randn(n + 1, Hkv, D, generator=g, dtype=torch.float64) for n in lens]
    n_pages = 64
    k_pool = torch.zeros(n_pages, P, Hkv, D, dtype=torch.float64)
    v_pool = torch.zeros_like(k_pool)
    cs = O.build_cos_sin_cache(D, 256, base).double()
    # an exact fp64 table so the closed form and the table path share their angles
    inv = 1.0 / (torch.tensor(base, dtype=torch.float64) ** (torch.arange(0, D, 2, dtype=torch.float64) / D))
    ang = torch.arange(256, dtype=torch.float64)[:, None] * inv[None, :]
    cs = torch.cat([ang.cos(), ang.sin()], dim=-1)
    rope = O.RopeSpec(D, cs)
    blocks, page = [], 0
    for j, n in enumerate(lens):
        b = O.OBlock(P)
        if n:
            npg = -(-n // P)
            b.grow_pages([(page + i) * P for i in range(npg)], n)
            page += npg
            slots = torch.tensor(b.token_slots())
            k_rot = rope.rotate(raw_k[j][:n], torch.arange(n))
            k_pool.view(-1, Hkv, D)[slots] = k_rot
            v_pool.view(-1, Hkv, D)[slots] = val[j][:n]
        blocks.append(b)
    return dict(Hq=Hq, Hkv=Hkv, D=D, base=base, lens=lens, raw_k=raw_k, val=val, k_pool=k_pool, v_pool=v_pool,
                rope=rope, blocks=blocks, next_page=page, gen=g)


@pytest.mark.parametrize("P", [1, 4])
@pytest.mark.parametrize("aux", [False, True])
def test_decode_equals_one_softmax_over_concatenated_view(P, aux):
    c = _random_view_case(7, P, aux, False)
    blocks, Hq, Hkv, D = c["blocks"], c["Hq"], c["Hkv"], c["D"]
    writer = blocks[3]
    view = [blocks[0], blocks[1], blocks[2], blocks[0]] if aux else [blocks[0], blocks[1], blocks[2], blocks[3], blocks[0]]
    pending, slots, pos = O.plan_decode_writes([writer], P, lambda n: [(c["next_page"] + i) * P for i in range(n)])
    plan = O.plan_decode([view], [writer], pending, slots, P)
    # store the new token (block index 3, position = its span)
    j, n = 3, c["lens"][3]
    k_new = c["rope"].rotate(c["raw_k"][j][n:n + 1], torch.tensor([pos[0]]))
    O.store_kv(c["k_pool"].view(-1, Hkv * D), c["v_pool"].view(-1, Hkv * D), torch.tensor(slots),
               k_new.reshape(1, -1), c["val"][j][n:n + 1].reshape(1, -1))
    q = torch.randn(1, Hq, D, generator=c["gen"], dtype=torch.float64)
    out, lse, _ = O.forward_decode(plan, q, c["k_pool"], c["v_pool"], c["rope"], math_dtype=torch.float64)
    # closed form: keys at absolute positions of the concatenation, query at the end
    order = [0, 1, 2, 0] if aux else [0, 1, 2, 3, 0]
    seg_len = [c["lens"][i] + (1 if i == 3 else 0) for i in order]
    starts, acc = [], 0
    for n_ in seg_len:
        starts.append(acc)
        acc += n_
    keys = [c["raw_k"][i][:n_] for i, n_ in zip(order, seg_len)]
    vals = [c["val"][i][:n_] for i, n_ in zip(order, seg_len)]
    rel = [torch.arange(n_) for n_ in seg_len]
    q_pos = acc - 1
    if aux:
        # the writer's own token is outside the view: it sits at the query's position
        keys.append(c["raw_k"][3][n:n + 1])
        vals.append(c["val"][3][n:n + 1])
        starts.append(acc)
        rel.append(torch.arange(1))
        # the query is rotated per segment relative to segment starts; for the own token
        # the distance is 0 whatever absolute position is chosen, so compare scores only
        q_pos = acc
        # view total does not include the own token: distances to view keys grow by one
        starts = [s + 1 for s in starts[:-1]] + [acc]
    want, wlse = O.concat_view_attention(q[0], q_pos, keys, vals, starts, rel, D, c["base"])
    assert torch.allclose(out.view(Hq, D), want, atol=1e-10)
    assert torch.allclose(lse[0], wlse, atol=1e-10)


def test_prefill_equals_one_causal_softmax_over_concatenated_view():
    P = 4
    c = _random_view_case(8, P, False, False)
    blocks, Hq, Hkv, D, g = c["blocks"], c["Hq"], c["Hkv"], c["D"], c["gen"]
    ctx = [blocks[0], blocks[2]]
    T, S = c["lens"][3], 6  # the write block already holds 3 tokens
    raw_new = torch.randn(S, Hkv, D, generator=g, dtype=torch.float64)
    val_new = torch.randn(S, Hkv, D, generator=g, dtype=torch.float64)
    own = blocks[3]
    fresh = [(c["next_page"] + i) * P for i in range(own.pages_needed(S))]
    starts_all = own.page_starts + fresh
    slots = [starts_all[i // P] + i % P for i in range(T, T + S)]
    k_rot = c["rope"].rotate(raw_new, torch.arange(T, T + S))
    O.store_kv(c["k_pool"].view(-1, Hkv * D), c["v_pool"].view(-1, Hkv * D), torch.tensor(slots),
               k_rot.reshape(S, -1), val_new.reshape(S, -1))
    plan = O.plan_prefill_batch([O.OPrefillSpec(ctx, starts_all, S, T)], P)
    q = torch.randn(S, Hq, D, generator=g, dtype=torch.float64)
    out, lse = O.forward_prefill_batch(plan, q, c["k_pool"], c["v_pool"], c["rope"], math_dtype=torch.float64)
    L0, L2 = c["lens"][0], c["lens"][2]
    for u in range(S):
        keys = [c["raw_k"][0][:L0], c["raw_k"][2][:L2], torch.cat([c["raw_k"][3][:T], raw_new[:u + 1]])]
        vals = [c["val"][0][:L0], c["val"][2][:L2], torch.cat([c["val"][3][:T], val_new[:u + 1]])]
        starts = [0, L0, L0 + L2]
        rel = [torch.arange(k.shape[0]) for k in keys]
        want, wlse = O.concat_view_attention(q[u], L0 + L2 + T + u, keys, vals, starts, rel, D, c["base"])
        assert torch.allclose(out[u].view(Hq, D), want, atol=1e-10)
        assert torch.allclose(lse[u], wlse, atol=1e-10)


def test_zero_keys_unit_values_give_ones():
    P, Hq, Hkv, D = 16, 16, 2, 32
    k_pool = torch.zeros(8, P, Hkv, D)
    v_pool = torch.ones(8, P, Hkv, D)
    b = O.OBlock(P, [0, P], 31)
    plan = O.plan_decode([[b]], [b], {id(b): None}, [31], P)
    rope = O.RopeSpec(D, O.build_cos_sin_cache(D, 64, 1e4))
    out, lse, _ = O.forward_decode(plan, torch.randn(1, Hq, D), k_pool, v_pool, rope)
    assert torch.allclose(out, torch.ones_like(out), atol=1e-6)
    assert torch.allclose(lse, torch.full_like(lse, math.log(32)), atol=1e-5)
