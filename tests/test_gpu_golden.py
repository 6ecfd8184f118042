"""GPU parity against the committed fp64 closed-form answers
(tests/golden/view_attention_fp64.npz): the product op on the HIP path, from
unrotated inputs to outputs and LSE, in fp32 (vector-ALU kernel) and in bf16
(matrix-core kernels)."""

from types import SimpleNamespace

import pytest
import torch

from async_llm_amd.shared_cache import CacheBlock, PrefillSpec, SharedCacheAttention, WorkerGroup
from async_llm_amd.shared_cache.session_planning import plan_decode_writes
from tests import golden_cases as G
from tests.util import assert_close

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda")


class _FreePages:
    def __init__(self, pages, page_size):
        self.pages, self.page_size = list(pages), page_size

    def alloc_pages(self, n):
        out, self.pages = self.pages[:n], self.pages[n:]
        return torch.tensor([p * self.page_size for p in out], dtype=torch.int32)


def _setup(c, dtype, kernel):
    Hq, Hkv, D, P = c["Hq"], c["Hkv"], c["D"], c["P"]
    k_pool, v_pool, pages, free, rope, table = G.lay_out(c, dtype)
    k_dev, v_dev = k_pool.to(DEV), v_pool.to(DEV)
    pool = SimpleNamespace(k_cache=lambda layer: k_dev, v_cache=lambda layer: v_dev)
    op = SharedCacheAttention(pool, table.to(DEV), Hq, Hkv, D, P, dtype, DEV, kernel=kernel)
    blocks = []
    for pg, n in zip(pages, c["lens"]):
        b = CacheBlock(DEV, P)
        if n:
            b.grow_pages(torch.tensor([p * P for p in pg]), n)
        blocks.append(b)
    return op, blocks, _FreePages(free, P)


@pytest.mark.parametrize("dtype,kernel", [(torch.float32, "generic"), (torch.bfloat16, "auto"), (torch.bfloat16, "generic")])
@pytest.mark.parametrize("aux", [False, True])
def test_decode_matches_the_closed_form_answers(dtype, kernel, aux):
    c = G.load()
    Hq, Hkv, D, P = c["Hq"], c["Hkv"], c["D"], c["P"]
    op, b, free = _setup(c, dtype, kernel)
    view = [b[0], b[1], b[2], b[0]] if aux else [b[0], b[1], b[2], b[3], b[0]]
    group = WorkerGroup(cache_structure=[view], write_to=[b[3]])
    pending, slots, pos = plan_decode_writes(group, P, free, DEV)
    meta = op.prepare(group, pending, slots)
    n = c["lens"][3]
    batch = SimpleNamespace(attn_metadata=meta, positions=torch.tensor(pos, dtype=torch.int64, device=DEV), out_loc=slots,
                            mrope_positions=None)
    q = c["q_dec"].reshape(1, Hq * D).to(dtype).to(DEV)
    k = c["raw_k"][3][n:n + 1].reshape(1, Hkv * D).to(dtype).to(DEV)  # UNROTATED: the op rotates and stores it
    v = c["val"][3][n:n + 1].reshape(1, Hkv * D).to(dtype).to(DEV)
    out, lse = op.forward_with_lse(q, k, v, 0, batch)
    want, wlse = c["decode_aux" if aux else "decode"]
    assert_close(out.view(Hq, D), want, dtype, "out")
    assert_close(lse[0], wlse, dtype, "lse")


@pytest.mark.parametrize("dtype,kernel", [(torch.float32, "generic"), (torch.bfloat16, "auto"), (torch.float16, "auto")])
def test_prefill_matches_the_closed_form_answers(dtype, kernel):
    c = G.load()
    Hq, Hkv, D, P, S, T = c["Hq"], c["Hkv"], c["D"], c["P"], c["S"], c["lens"][3]
    op, b, free = _setup(c, dtype, kernel)
    own = b[3]
    fresh = free.alloc_pages(own.pages_needed(S))
    starts_all = torch.tensor(list(own.page_starts) + fresh.tolist(), dtype=torch.int32)
    meta = op.prepare_prefill_batch([PrefillSpec([b[0], b[2]], starts_all, S, T)])
    slots = (starts_all.to(torch.int64)[:, None] + torch.arange(P)[None, :]).reshape(-1)[T:T + S].to(torch.int32)
    batch = SimpleNamespace(attn_metadata=meta, positions=torch.arange(T, T + S, device=DEV), out_loc=slots.to(DEV),
                            mrope_positions=None)
    q = c["q_pre"].reshape(S, Hq * D).to(dtype).to(DEV)
    k = c["raw_k"][3][T:T + S].reshape(S, Hkv * D).to(dtype).to(DEV)
    v = c["val"][3][T:T + S].reshape(S, Hkv * D).to(dtype).to(DEV)
    out, lse = op.forward_with_lse(q, k, v, 0, batch)
    want, wlse = c["prefill"]
    assert_close(out.view(S, Hq, D), want, dtype, "out")
    assert_close(lse, wlse, dtype, "lse")
