"""``va_attention_static`` (the entry point that allocates nothing) against ``va_attention``:
the same plan, the same kernels, the partial states in the library's own per-GPU array instead
of a caller's workspace.  Results must be identical bit for bit, on two calls in a row of which
the second is smaller (the array keeps the first call's contents), and a plan whose partial
states exceed the array must be refused with a clear error."""

import pytest
import torch

from async_llm_amd import native, workloads

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda")


def _both_ways(wl):
    op, meta = wl.op, wl.meta
    counts = meta.launch.counts
    assert counts.n_partials > 0, "the workload must split rows over work items, or no scratch is used"
    assert counts.workspace_bytes <= native.STATIC_SCRATCH_BYTES
    op.store_new_kv(wl.k, wl.v, 0, wl.batch)
    want, want_lse = op.attend(wl.q, 0, meta, return_lse=True)
    W, Hq, D = meta.num_workers, op.num_qo_heads, op.head_dim
    out = torch.full((W, Hq * D), float("nan"), dtype=op.dtype, device=DEV)
    lse = torch.full((W, Hq), float("nan"), dtype=torch.float32, device=DEV)
    # one call first: the once-per-device lookup of the array's address (and whatever the runtime
    # sets up lazily for a kernel's first launch) is kept apart from the steady-state call measured below
    op.attend(wl.q, 0, meta, return_lse=True, out=out, lse=lse, static_scratch=True)
    out.fill_(float("nan"))
    lse.fill_(float("nan"))
    torch.cuda.synchronize()
    before = torch.cuda.memory_stats(DEV)["allocation.all.allocated"]
    free_before, _ = torch.cuda.mem_get_info(DEV)
    got, got_lse = op.attend(wl.q, 0, meta, return_lse=True, out=out, lse=lse, static_scratch=True)
    assert torch.cuda.memory_stats(DEV)["allocation.all.allocated"] == before  # torch allocated nothing either
    torch.cuda.synchronize()
    # ... and neither did the library behind torch's back: the device's free memory is what it was
    free_after, _ = torch.cuda.mem_get_info(DEV)
    assert free_after == free_before, f"device memory in use changed by {free_before - free_after} bytes"
    assert got.data_ptr() == out.data_ptr()
    assert torch.equal(got, want) and torch.equal(got_lse, want_lse)
    return counts.workspace_bytes


def test_static_scratch_matches_the_workspace_path_twice_in_a_row():
    # 24 requests over a shared block: a few hundred partial states of 16 heads x (256 + 2) floats
    big = _both_ways(workloads.batched_decode(DEV, workers=24, shared_len=4096, private_lo=200, private_hi=3000))
    # then a smaller launch (other head layout, other plan) over the same array
    small = _both_ways(workloads.batched_decode(DEV, workers=3, shared_len=900, private_lo=40, private_hi=700,
                                                heads=(8, 2, 128), seed=7))
    assert small < big
    # and a prefill whose tiles are split by tokens (partial states written by the wide kernel)
    _both_ways(workloads.view_prefill(DEV, requests=1, new_tokens=64, own_prefix=32, prompt_len=6000))


def test_static_scratch_refuses_a_plan_that_does_not_fit():
    wl = workloads.mixed_batch(DEV, decode_rows=8, chunks=2, chunk_len=512, ctx_lo=20000, ctx_hi=30000)
    op, meta = wl.op, wl.meta
    assert meta.launch.counts.workspace_bytes > native.STATIC_SCRATCH_BYTES
    out = torch.empty((meta.num_workers, op.num_qo_heads * op.head_dim), dtype=op.dtype, device=DEV)
    with pytest.raises(native.ViewAttnError, match="va_attention_static.*scratch"):
        op.attend(wl.q, 0, meta, out=out, static_scratch=True)
    op.attend(wl.q, 0, meta, out=out)  # the workspace path takes it
    torch.cuda.synchronize()
