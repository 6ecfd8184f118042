"""q, k and v as row-strided slices of ONE fused projection output, which is how the
reference's attention layers hand them to the op (``layers/attention.py:47-64``:
``qkv.split(...)`` views, then ``sc_op.forward(q, k, v, ...)``): every attention kernel
(streaming and wide matrix-core kernels, vector-ALU kernel) and the rotate+store kernel
must honour the row stride.  The columns between and behind the slices are NaN."""

import pytest
import torch

from async_llm_amd.shared_cache import CacheBlock, PrefillSpec, WorkerGroup
from tests.test_gpu_decode import Pages
from tests.util import make_op_and_pool, run_decode_parity, run_prefill_parity

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda")


@pytest.mark.parametrize("kernel,dtype,heads", [
    ("auto", torch.bfloat16, (16, 4, 256)),   # streaming matrix-core kernel, 16-row tiles of 4 requests x 4 heads
    ("auto", torch.float16, (8, 2, 128)),
    ("generic", torch.bfloat16, (8, 2, 64)),  # vector-ALU kernel
    ("auto", torch.float32, (8, 2, 128)),     # fp32: always the vector-ALU kernel
])
def test_decode_with_fused_qkv_rows(kernel, dtype, heads):
    page = 16
    op, cpu_pool, dev_pool, gen = make_op_and_pool(DEV, dtype, heads, page, 400, 1e4, seed=91, kernel=kernel)
    pages = Pages(page)
    shared = pages.block(700)
    private = [pages.block(n) for n in (33, 260, 17, 1200, 64)]
    group = WorkerGroup(cache_structure=[[shared, b] for b in private], write_to=private)
    out, lse, exp_out, exp_lse, meta = run_decode_parity(op, cpu_pool, dev_pool, group, pages, 1e4, gen, fused_qkv=True)
    assert torch.isfinite(out.float()).all() and torch.isfinite(lse).all()
    want = 2 if kernel == "auto" and dtype != torch.float32 else 1
    assert meta.launch.counts.kernel == want


@pytest.mark.parametrize("kernel,dtype,heads", [
    ("auto", torch.bfloat16, (16, 4, 256)),  # wide matrix-core kernel (128-row tiles) + streaming kernel for the tails
    ("auto", torch.float16, (8, 2, 64)),
    ("generic", torch.float32, (4, 2, 64)),
])
def test_prefill_with_fused_qkv_rows(kernel, dtype, heads):
    page = 16
    op, cpu_pool, dev_pool, gen = make_op_and_pool(DEV, dtype, heads, page, 300, 1e4, seed=92, kernel=kernel, max_pos=4096)
    context = []
    for start, length in ((0, 300), (20, 77)):
        b = CacheBlock(DEV, page)
        b.grow_pages(torch.arange(start, start + -(-length // page)) * page, length)
        context.append(b)
    specs = []
    for r, (new, prefix) in enumerate(((70, 5), (33, 0), (129, 40))):
        first = 30 + r * 15
        starts = torch.arange(first, first + -(-(prefix + new) // page), dtype=torch.int32) * page
        specs.append(PrefillSpec(context[: 2 - r % 2], starts, new, prefix))
    out, lse, exp_out, exp_lse, meta = run_prefill_parity(op, cpu_pool, dev_pool, specs, 1e4, gen, fused_qkv=True)
    assert torch.isfinite(out.float()).all() and torch.isfinite(lse).all()
    if kernel == "auto":
        assert meta.launch.counts.n_wide_items > 0 and meta.launch.counts.n_items > meta.launch.counts.n_wide_items
