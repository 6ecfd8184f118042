"""Writes tests/golden/view_attention_fp64.npz: small seeded cache-view attention
cases with answers from the fp64 closed form (ONE softmax over the concatenated
view, keys at absolute positions, RoPE from its definition) -- no paged layout,
no per-segment evaluation, no merge, no rotation table.

    python tests/golden/make_view_attention_fixture.py

Inputs are bf16 values (stored as their 16-bit patterns), so the same arrays feed
fp32 and bf16 runs without further input rounding; answers are float64.  Cases:
  decode      view [b0, b1(empty), b2, b3, b0], the writer b3 is in the view and appends one token
  decode_aux  view [b0, b1, b2, b0], the writer b3 is NOT in the view (its own token is a segment)
  prefill     context [b0, b2], the request's block b3 holds T tokens and gets S new ones
"""

import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import view_attention_oracle as O  # noqa: E402

HQ, HKV, D, BASE, P = 8, 2, 64, 1e4, 4
LENS = [21, 0, 16 + 5, 9]  # tokens already in blocks b0..b3
S_NEW = 11  # new tokens of the prefill case


def bf16_round(x):
    return x.to(torch.bfloat16).to(torch.float32)


def bits(x):
    """bf16 bit patterns of an fp32 tensor that holds bf16 values."""
    return x.to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)


def main():
    g = torch.Generator().manual_seed(20240607)
    scale = D ** -0.25  # keeps scores O(1) after the 1/sqrt(D) of the attention
    extra = [0, 0, 0, S_NEW]  # only the written block b3 gets new tokens
    raw_k = [bf16_round(torch.randn(n + e, HKV, D, generator=g) * scale) for n, e in zip(LENS, extra)]
    val = [bf16_round(torch.randn(n + e, HKV, D, generator=g)) for n, e in zip(LENS, extra)]
    q_dec = bf16_round(torch.randn(1, HQ, D, generator=g) * scale)
    q_pre = bf16_round(torch.randn(S_NEW, HQ, D, generator=g) * scale)
    out = dict(hq=HQ, hkv=HKV, d=D, base=BASE, page=P, lens=np.array(LENS), s_new=S_NEW, q_dec=bits(q_dec),
               q_pre=bits(q_pre))
    for j in range(4):
        out[f"raw_k{j}"] = bits(raw_k[j])
        out[f"val{j}"] = bits(val[j])

    def closed_form(q_row, q_pos, order, seg_len, extra=None, shift=0):
        starts, acc = [], 0
        for n in seg_len:
            starts.append(acc + shift)
            acc += n
        keys = [raw_k[i][:n] for i, n in zip(order, seg_len)]
        vals = [val[i][:n] for i, n in zip(order, seg_len)]
        rel = [torch.arange(n) for n in seg_len]
        if extra is not None:
            keys.append(extra[0]); vals.append(extra[1]); starts.append(extra[2]); rel.append(torch.arange(1))
        return O.concat_view_attention(q_row, q_pos, keys, vals, starts, rel, D, BASE)

    # decode: the writer (b3) is in the view; its new token is token LENS[3] of b3
    order = [0, 1, 2, 3, 0]
    seg = [LENS[i] + (1 if i == 3 else 0) for i in order]
    o, l = closed_form(q_dec[0], sum(seg) - 1, order, seg)
    out["decode_out"], out["decode_lse"] = o.numpy(), l.numpy()

    # decode_aux: the writer is outside the view; its token sits at the query's own position
    order = [0, 1, 2, 0]
    seg = [LENS[i] for i in order]
    total = sum(seg)
    n3 = LENS[3]
    o, l = closed_form(q_dec[0], total, order, seg, extra=(raw_k[3][n3:n3 + 1], val[3][n3:n3 + 1], total), shift=1)
    out["decode_aux_out"], out["decode_aux_lse"] = o.numpy(), l.numpy()

    # prefill: context [b0, b2] then the own block (T old + causal new tokens)
    T = LENS[3]
    L0, L2 = LENS[0], LENS[2]
    outs, lses = [], []
    for u in range(S_NEW):
        keys = [raw_k[0][:L0], raw_k[2][:L2], raw_k[3][:T + u + 1]]
        vals = [val[0][:L0], val[2][:L2], val[3][:T + u + 1]]
        rel = [torch.arange(k.shape[0]) for k in keys]
        o, l = O.concat_view_attention(q_pre[u], L0 + L2 + T + u, keys, vals, [0, L0, L0 + L2], rel, D, BASE)
        outs.append(o); lses.append(l)
    out["prefill_out"], out["prefill_lse"] = torch.stack(outs).numpy(), torch.stack(lses).numpy()

    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "view_attention_fp64.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
