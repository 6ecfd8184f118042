"""The CPU oracle (paged layout, per-segment attention, LSE merge, table RoPE,
fp32 math) against the committed fp64 closed-form answers of
tests/golden/view_attention_fp64.npz."""

import torch

from oracle import view_attention_oracle as O
from tests import golden_cases as G


def _blocks(c, pages):
    P = c["P"]
    return [O.OBlock(P, [p * P for p in pg], n) for pg, n in zip(pages, c["lens"])]


def _decode(c, aux):
    Hq, Hkv, D, P = c["Hq"], c["Hkv"], c["D"], c["P"]
    k_pool, v_pool, pages, free, rope, _ = G.lay_out(c, torch.float32)
    b = _blocks(c, pages)
    writer = b[3]
    view = [b[0], b[1], b[2], b[0]] if aux else [b[0], b[1], b[2], b[3], b[0]]
    free_iter = iter(free)
    pending, slots, pos = O.plan_decode_writes([writer], P, lambda n: [next(free_iter) * P for _ in range(n)])
    plan = O.plan_decode([view], [writer], pending, slots, P)
    n = c["lens"][3]
    k_new = rope.rotate(c["raw_k"][3][n:n + 1], torch.tensor([pos[0]]))
    O.store_kv(k_pool.view(-1, Hkv * D), v_pool.view(-1, Hkv * D), torch.tensor(slots), k_new.reshape(1, -1),
               c["val"][3][n:n + 1].reshape(1, -1))
    out, lse, _ = O.forward_decode(plan, c["q_dec"], k_pool, v_pool, rope)
    return out.view(Hq, D), lse[0]


def test_decode_matches_the_closed_form_answers():
    c = G.load()
    for aux, name in ((False, "decode"), (True, "decode_aux")):
        out, lse = _decode(c, aux)
        want, wlse = c[name]
        assert torch.allclose(out.double(), want, atol=2e-5, rtol=1e-5), name
        assert torch.allclose(lse.double(), wlse, atol=2e-5, rtol=1e-5), name


def test_prefill_matches_the_closed_form_answers():
    c = G.load()
    Hq, Hkv, D, P, S, T = c["Hq"], c["Hkv"], c["D"], c["P"], c["S"], c["lens"][3]
    k_pool, v_pool, pages, free, rope, _ = G.lay_out(c, torch.float32)
    b = _blocks(c, pages)
    own = b[3]
    starts_all = own.page_starts + [p * P for p in free[: own.pages_needed(S)]]
    slots = [starts_all[i // P] + i % P for i in range(T, T + S)]
    k_rot = rope.rotate(c["raw_k"][3][T:T + S], torch.arange(T, T + S))
    O.store_kv(k_pool.view(-1, Hkv * D), v_pool.view(-1, Hkv * D), torch.tensor(slots), k_rot.reshape(S, -1),
               c["val"][3][T:T + S].reshape(S, -1))
    plan = O.plan_prefill_batch([O.OPrefillSpec([b[0], b[2]], starts_all, S, T)], P)
    out, lse = O.forward_prefill_batch(plan, c["q_pre"], k_pool, v_pool, rope)
    want, wlse = c["prefill"]
    assert torch.allclose(out.view(S, Hq, D).double(), want, atol=2e-5, rtol=1e-5)
    assert torch.allclose(lse.double(), wlse, atol=2e-5, rtol=1e-5)
