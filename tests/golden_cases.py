"""Loader of tests/golden/view_attention_fp64.npz (answers from the fp64 closed
form, see tests/golden/make_view_attention_fixture.py) and builders that lay the
fixture's blocks out in a paged pool."""

from __future__ import annotations

import os

import numpy as np
import torch

from oracle import view_attention_oracle as O

PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "view_attention_fp64.npz")


def _bf16(bits: np.ndarray) -> torch.Tensor:
    return torch.from_numpy(bits.view(np.int16).copy()).view(torch.bfloat16).to(torch.float32)


def load():
    z = np.load(PATH)  # plain arrays only (allow_pickle stays False)
    c = dict(Hq=int(z["hq"]), Hkv=int(z["hkv"]), D=int(z["d"]), base=float(z["base"]), P=int(z["page"]),
             lens=[int(x) for x in z["lens"]], S=int(z["s_new"]), q_dec=_bf16(z["q_dec"]), q_pre=_bf16(z["q_pre"]))
    c["raw_k"] = [_bf16(z[f"raw_k{j}"]) for j in range(4)]
    c["val"] = [_bf16(z[f"val{j}"]) for j in range(4)]
    for name in ("decode", "decode_aux", "prefill"):
        c[name] = (torch.from_numpy(z[name + "_out"]), torch.from_numpy(z[name + "_lse"]))
    return c


def lay_out(c, dtype, num_pages=64):
    """Pool with the blocks' old tokens stored (keys rotated to block-relative
    positions by the oracle's table path) on a scattered page list; returns
    (k_pool, v_pool, page lists per block, first unused page, rope)."""
    Hkv, D, P = c["Hkv"], c["D"], c["P"]
    table = O.build_cos_sin_cache(D, 512, c["base"])
    rope = O.RopeSpec(D, table)
    k_pool = torch.zeros(num_pages, P, Hkv, D, dtype=dtype)
    v_pool = torch.zeros_like(k_pool)
    order = torch.randperm(num_pages, generator=torch.Generator().manual_seed(5)).tolist()
    pages, used = [], 0
    for j, n in enumerate(c["lens"]):
        npg = -(-n // P)
        mine = order[used: used + npg]
        used += npg
        pages.append(mine)
        if n:
            slots = torch.tensor([mine[i // P] * P + i % P for i in range(n)])
            k_rot = rope.rotate(c["raw_k"][j][:n].to(dtype), torch.arange(n))
            k_pool.view(-1, Hkv, D)[slots] = k_rot.to(dtype)
            v_pool.view(-1, Hkv, D)[slots] = c["val"][j][:n].to(dtype)
    return k_pool, v_pool, pages, order[used:], rope, table
