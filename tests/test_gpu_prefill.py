"""GPU parity of view-conditioned prefill: product op vs the CPU oracle.
Scenarios follow tests/core/test_shared_prefill_attention_graph.py:14-135 of
the reference (ragged requests, 0..3 context blocks, non-empty write blocks,
3-D mRoPE positions on some requests) plus scaled configuration 3."""

import pytest
import torch

from async_llm_amd import workloads
from async_llm_amd.shared_cache import CacheBlock, PrefillSpec
from oracle import view_attention_oracle as O
from tests.util import assert_close, make_op_and_pool, oracle_prefill_plan, oracle_rope, run_prefill_parity

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda")
KERNELS = ["generic", "auto"]


def common_blocks(page, mrope):
    blocks = []
    for start, length in zip((0, 2, 5), (17, 35, 9)):
        b = CacheBlock(DEV, page)
        b.grow_pages(torch.arange(start, start + -(-length // page)) * page, length)
        if mrope:
            b.mrope_span_override = length // 2 + 1
        blocks.append(b)
    return blocks


def make_specs(common, lengths, turn, page, mrope, full_context=False, depth=3):
    specs = []
    for worker, length in enumerate(lengths):
        prefix = (worker * 7 + turn) % 14
        pages = torch.arange(10 + worker * 12, 10 + worker * 12 + -(-(prefix + length) // page), dtype=torch.int32) * page
        rel = None
        if mrope and (worker + turn) % 2:
            p = torch.arange(length)
            rel = torch.stack([p // 8, p // 4, p % 4])
        own_span = prefix // 2 if mrope else prefix
        context = [common[(turn + j) % 3] for j in range(depth if full_context else (worker + turn) % 4)]
        specs.append(PrefillSpec(context, pages, length, prefix, own_span, rel))
    return specs


@pytest.mark.parametrize("kernel", KERNELS)
@pytest.mark.parametrize("mrope", [False, True])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_ragged_prefill_batches(kernel, mrope, dtype):
    page, heads = 16, (4, 2, 64)
    op, cpu_pool, dev_pool, gen = make_op_and_pool(
        DEV, dtype, heads, page, 64, 1e4, rotary_dim=32 if mrope else 64,
        mrope_section=(8, 4, 4) if mrope else None, seed=734, scale=1.0, kernel=kernel, max_pos=2048)
    common = common_blocks(page, mrope)
    for turn, lengths in ((0, [1]), (2, [63, 65, 3]), (3, [138, 91, 1]), (4, [64] * 4), (5, [9, 7])):
        specs = make_specs(common, lengths, turn, page, mrope, full_context=(turn == 4))
        run_prefill_parity(op, cpu_pool, dev_pool, specs, 1e4, gen, scale=1.0)


@pytest.mark.parametrize("kernel", KERNELS)
def test_plain_prefill_without_context(kernel):
    page = 16
    op, cpu_pool, dev_pool, gen = make_op_and_pool(DEV, torch.bfloat16, (8, 2, 128), page, 64, 1e6, seed=5,
                                                   kernel=kernel)
    specs = [PrefillSpec([], torch.arange(0, 9, dtype=torch.int32) * page, 130),
             PrefillSpec([], torch.arange(20, 22, dtype=torch.int32) * page, 5, 20)]
    *_, meta = run_prefill_parity(op, cpu_pool, dev_pool, specs, 1e6, gen)
    assert meta.n_ctx_rows == 0 and meta.max_segments == 1


@pytest.mark.parametrize("kernel", KERNELS)
def test_scaled_view_prefill_configuration(kernel):
    """Configuration 3 at reduced size: every request extends its own block and
    reads the prompt plus the other requests' blocks at their pre-write length."""
    wl = workloads.view_prefill(DEV, requests=3, new_tokens=96, own_prefix=40, prompt_len=300, kernel=kernel)
    op = wl.op
    Hq, Hkv, D, P = op.num_qo_heads, op.num_kv_heads, op.head_dim, op.page_size
    k_cpu, v_cpu = wl.pool.k_cache(0).cpu(), wl.pool.v_cache(0).cpu()
    out, lse = op.forward_with_lse(wl.q, wl.k, wl.v, 0, wl.batch)
    oplan = oracle_prefill_plan(wl.specs, P)
    assert torch.equal(wl.meta.sub_loc.cpu(), oplan.sub_loc)
    rope = oracle_rope(op, wl.theta)
    N = wl.q.shape[0]
    k_rot = rope.rotate(wl.k.cpu().view(N, Hkv, D), wl.batch.positions.cpu())
    O.store_kv(k_cpu.view(-1, Hkv * D), v_cpu.view(-1, Hkv * D), wl.batch.out_loc.cpu(), k_rot.reshape(N, -1), wl.v.cpu())
    assert torch.equal(wl.pool.k_cache(0).cpu(), k_cpu)
    eo, el = O.forward_prefill_batch(oplan, wl.q.cpu().view(N, Hq, D), k_cpu, v_cpu, rope)
    assert_close(out, eo, op.dtype, "out")
    assert_close(lse, el, op.dtype, "lse")
    pairs = 3 * (96 * (300 + 2 * 40) + 96 * 40 + 96 * 97 // 2)
    assert wl.alg_flops == 4 * D * Hq * pairs
    assert wl.meta.last_indices.tolist() == [95, 191, 287]


@pytest.mark.parametrize("kernel", KERNELS)
def test_mixed_batch_single_launch(kernel):
    """Configuration 4 at reduced size: decode rows and prefill chunks planned and
    run as ONE launch; each part must equal its own oracle evaluation over the
    pool after ALL new rows were stored."""
    from tests.util import oracle_decode_plan

    wl = workloads.mixed_batch(DEV, decode_rows=5, chunks=2, chunk_len=40, ctx_lo=100, ctx_hi=900, shared_len=70,
                               kernel=kernel)
    op, meta = wl.op, wl.meta
    Hq, Hkv, D, P = op.num_qo_heads, op.num_kv_heads, op.head_dim, op.page_size
    W, N = 5, 5 + 2 * 40
    assert meta.phase == "mixed" and meta.num_workers == N
    assert meta.get_last_indices(0).tolist() == [0, 1, 2, 3, 4, 5 + 39, 5 + 79]
    assert len(set(meta.pad_slot.tolist())) == meta.pad_slot.numel()
    k_cpu, v_cpu = wl.pool.k_cache(0).cpu(), wl.pool.v_cache(0).cpu()
    out, lse = op.forward_with_lse(wl.q, wl.k, wl.v, 0, wl.batch)
    rope = oracle_rope(op, wl.theta)
    k_rot = rope.rotate(wl.k.cpu().view(N, Hkv, D), wl.batch.positions.cpu())
    O.store_kv(k_cpu.view(-1, Hkv * D), v_cpu.view(-1, Hkv * D), wl.batch.out_loc.cpu(), k_rot.reshape(N, -1), wl.v.cpu())
    assert torch.equal(wl.pool.k_cache(0).cpu(), k_cpu) and torch.equal(wl.pool.v_cache(0).cpu(), v_cpu)
    dplan = oracle_decode_plan(wl.group, wl.pending, wl.new_token_slots.cpu(), P)
    pplan = oracle_prefill_plan(wl.specs, P)
    assert meta.sub_loc.tolist() == dplan.sub_loc + pplan.sub_loc.tolist()
    assert meta.sub_worker.tolist() == dplan.sub_worker + [r + W for r in pplan.sub_worker]
    q_cpu = wl.q.cpu().view(N, Hq, D)
    eo_d, el_d, _ = O.forward_decode(dplan, q_cpu[:W], k_cpu, v_cpu, rope)
    eo_p, el_p = O.forward_prefill_batch(pplan, q_cpu[W:], k_cpu, v_cpu, rope)
    assert_close(out[:W], eo_d, op.dtype, "decode rows")
    assert_close(lse[:W], el_d, op.dtype, "decode lse")
    assert_close(out[W:], eo_p, op.dtype, "prefill rows")
    assert_close(lse[W:], el_p, op.dtype, "prefill lse")


@pytest.mark.parametrize("page", [16, 4])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_split_chains(dtype, page):
    """Few query tiles over long context: the planner cuts each tile's chain of
    segments into several work items.  With pages of 16 tokens its cuts stay on
    16-token boundaries inside a segment (such pieces are fetched with uniform
    loads); with smaller pages they fall where the token budget ends, segment
    lengths that are no multiples of 16 make later pieces start anywhere, and
    the kernels address them token by token."""
    from tests.test_native_abi_cpu import decode_plan

    heads = (8, 2, 128)
    op, cpu_pool, dev_pool, gen = make_op_and_pool(DEV, dtype, heads, page, 5200 // page, 1e6, seed=77, kernel="auto",
                                                   max_pos=8192)
    lengths = (1999, 1501, 777)
    context, first = [], 0
    for length in lengths:
        b = CacheBlock(DEV, page)
        n_pages = -(-length // page)
        b.grow_pages(torch.arange(first, first + n_pages) * page, length)
        first += n_pages
        context.append(b)
    for new_tokens in (24, 3):  # a wide tile, then a narrow one
        pages = torch.arange(first, first + 64 // page, dtype=torch.int32) * page
        specs = [PrefillSpec(context, pages, new_tokens, 21)]
        *_, meta = run_prefill_parity(op, cpu_pool, dev_pool, specs, 1e6, gen)
        h, items, links, *_ = decode_plan(meta.launch.blob.cpu().numpy())
        real = [it for it in items if it[2] > 0]
        assert len(real) > 1, "the chain was not split"
        starts = [l[1] for it in real for l in links[it[0]: it[0] + it[1]]]
        if page >= 16:
            assert all(t % 16 == 0 for t in starts), "a cut left its 16-token boundary"
        else:
            assert any(t % 16 for t in starts), "no unaligned piece in this plan"


@pytest.mark.parametrize("dtype,heads,rotary", [
    (torch.bfloat16, (4, 4, 64), 64),      # one q head per kv head: 256-row wide tiles
    (torch.bfloat16, (16, 2, 128), 64),    # 8 q heads per kv head, partial rotation
    (torch.float16, (16, 1, 256), 256),    # 16 q heads per kv head: a wide tile is 8 requests rows
    (torch.float16, (8, 4, 256), 128),     # 2 q heads per kv head at head_dim 256
])
def test_prefill_head_layouts(dtype, heads, rotary):
    """Every supported ratio of q to kv heads through the wide and the streaming
    kernel: tiles of 256/G (128/G at head_dim 256) rows, tails of at most 16/G."""
    page = 16
    op, cpu_pool, dev_pool, gen = make_op_and_pool(DEV, dtype, heads, page, 96, 1e4, rotary_dim=rotary, seed=91,
                                                   scale=1.0, max_pos=2048)
    common = common_blocks(page, False)
    for turn, lengths in ((1, [170, 7]), (2, [33, 129, 1])):
        specs = make_specs(common, lengths, turn, page, False)
        *_, meta = run_prefill_parity(op, cpu_pool, dev_pool, specs, 1e4, gen, scale=1.0)
        assert meta.launch.counts.kernel == 2 and meta.launch.counts.n_wide_items > 0


@pytest.mark.parametrize("dtype,heads,rotary,mrope", [
    (torch.bfloat16, (8, 2, 256), 256, False),
    (torch.float16, (8, 4, 128), 64, False),
    (torch.bfloat16, (4, 2, 64), 64, False),
    (torch.bfloat16, (8, 2, 256), 128, True),
])
def test_long_links_of_whole_pages(dtype, heads, rotary, mrope):
    """Context blocks of hundreds of tokens on 16-token pages: the wide kernel walks
    the interior tiles of such a link with its branch-free ring step (page lookup
    a step ahead, uniform loads), the first, masked and last tiles with the
    general one.  Unit-variance data makes the per-row reference maxima rise
    inside those runs too (rescale and resume in the middle of a link)."""
    page = 16
    op, cpu_pool, dev_pool, gen = make_op_and_pool(
        DEV, dtype, heads, page, 200, 1e4, rotary_dim=rotary, mrope_section=(32, 16, 16) if mrope else None,
        seed=4242, scale=1.0 if heads[2] <= 64 else 0.5, max_pos=4096)
    blocks, first = [], 0
    for length in (701, 333, 96):
        b = CacheBlock(DEV, page)
        n_pages = -(-length // page)
        b.grow_pages(torch.arange(first, first + n_pages) * page, length)
        if mrope:
            b.mrope_span_override = length // 3 + 5
        blocks.append(b)
        first += n_pages
    specs = []
    for worker, (length, prefix) in enumerate(((96, 200), (17, 330))):
        n_pages = -(-(prefix + length) // page)
        pages = torch.arange(first, first + n_pages, dtype=torch.int32) * page
        first += n_pages
        rel = None
        if mrope and worker == 0:
            p = torch.arange(length)
            rel = torch.stack([p // 8, p // 4, p % 4])
        specs.append(PrefillSpec(blocks[worker:], pages, length, prefix, prefix // 2 if mrope else prefix, rel))
    assert first <= 200
    *_, meta = run_prefill_parity(op, cpu_pool, dev_pool, specs, 1e4, gen, scale=1.0 if heads[2] <= 64 else 0.5)
    assert meta.launch.counts.kernel == 2 and meta.launch.counts.n_wide_items > 0


@pytest.mark.parametrize("spike", [13.0, 15.0, 40.0])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("D", [64, 128, 256])
def test_wide_tiles_with_a_late_score_spike(D, dtype, spike):
    """The wide kernel keeps a per-row reference maximum and raises it in the middle of a segment
    only when a later tile exceeds it by more than 14 (log2 units).  Random N(0,1) scores never do,
    so here single keys are planted whose score is ``spike`` log2 units for every query row: one in
    an interior tile of a context block (the branch-free part of the walk) and one among the new
    tokens (the masked tiles at the causal edge).  Only the dims past ``rotary_dim`` carry the
    spike, so no rotation touches it.  13 stays just under the threshold (P = 2^13 must survive the
    16-bit P operand), 15 is just over it; with 40 the other keys are random and the spike towers
    over their running maximum."""
    heads, page, rotary = (8, 2, D), 16, D // 2
    random_keys = spike > 20
    op, cpu_pool, dev_pool, gen = make_op_and_pool(DEV, dtype, heads, page, 96, 1e4, rotary_dim=rotary, seed=91,
                                                   scale=1.0, kernel="auto", max_pos=2048)
    a = spike * 2.0 / (D ** 0.5 * 1.4426950408889634)  # a * (D/2) / sqrt(D) * log2(e) == spike
    if not random_keys:
        for pool in (cpu_pool[0], dev_pool[0]):
            pool.zero_()
    context = CacheBlock(DEV, page)
    context.grow_pages(torch.arange(0, 30) * page, 470)
    planted = 8 * page + 5  # token 213 of the context block (pages are in order here)
    for pool in (cpu_pool[0], dev_pool[0]):
        pool.view(-1, heads[1], D)[planted, :, :rotary] = 0
        pool.view(-1, heads[1], D)[planted, :, rotary:] = a
    new_tokens, prefix = 200, 24
    pages = torch.arange(40, 40 + -(-(prefix + new_tokens) // page), dtype=torch.int32) * page
    specs = [PrefillSpec([context], pages, new_tokens, prefix)]

    def mutate(q, k, v):
        q.view(-1, heads[0], D)[:, :, rotary:] = 1.0
        if not random_keys:
            k.zero_()
        k.view(-1, heads[1], D)[150, :, :rotary] = 0
        k.view(-1, heads[1], D)[150, :, rotary:] = a

    out, lse, exp_out, exp_lse, meta = run_prefill_parity(op, cpu_pool, dev_pool, specs, 1e4, gen, scale=1.0,
                                                          mutate=mutate)
    assert meta.launch.counts.n_wide_items > 0
    if not random_keys:  # every other score is 0: the closed form of the row's logsumexp
        seen = 470 + prefix + torch.arange(1, new_tokens + 1, dtype=torch.float64)
        spikes = 1 + (torch.arange(new_tokens) >= 150).double()
        a_stored = float(torch.tensor(a, dtype=dtype))  # the planted value as the pool holds it
        want = (seen - spikes + spikes * torch.tensor(a_stored * (D / 2) / D ** 0.5, dtype=torch.float64).exp()).log()
        got = lse.double().cpu()
        assert torch.allclose(got, want[:, None].expand_as(got), atol=2e-2, rtol=0)


@pytest.mark.parametrize("spike", [15.0, 60.0])
@pytest.mark.parametrize("dtype,D", [(torch.bfloat16, 256), (torch.float16, 128), (torch.bfloat16, 64)])
def test_wide_tiles_with_a_spike_in_the_first_tile_of_a_later_block(D, dtype, spike):
    """The reference maximum of a row is carried from block to block of a view (the score products of a tile
    start from minus that reference).  Here the first context block holds zero keys only, so the reference
    settles at 0, and the SECOND block opens with a key whose score is ``spike`` log2 units for every row: the
    raise happens on the first tile of a link, where no maxima were gathered ahead.  A third block of zero keys
    follows (scores far below the raised reference).  Closed form: every other score is 0."""
    heads, page, rotary = (8, 2, D), 16, D // 2
    op, cpu_pool, dev_pool, gen = make_op_and_pool(DEV, dtype, heads, page, 128, 1e4, rotary_dim=rotary, seed=17,
                                                   scale=1.0, kernel="auto", max_pos=4096)
    a = spike * 2.0 / (D ** 0.5 * 1.4426950408889634)
    for pool in (cpu_pool[0], dev_pool[0]):
        pool.zero_()
    blocks, first_page = [], 0
    for n in (256, 300, 130):
        b = CacheBlock(DEV, page)
        b.grow_pages(torch.arange(first_page, first_page + -(-n // page)) * page, n)
        first_page += -(-n // page)
        blocks.append(b)
    planted = (256 // page) * page + 3  # token 3 of the second block (pages are in order here)
    for pool in (cpu_pool[0], dev_pool[0]):
        pool.view(-1, heads[1], D)[planted, :, rotary:] = a
    new_tokens, prefix = 160, 16
    pages = torch.arange(60, 60 + -(-(prefix + new_tokens) // page), dtype=torch.int32) * page
    specs = [PrefillSpec(blocks, pages, new_tokens, prefix)]

    def mutate(q, k, v):
        q.view(-1, heads[0], D)[:, :, rotary:] = 1.0
        k.zero_()

    out, lse, exp_out, exp_lse, meta = run_prefill_parity(op, cpu_pool, dev_pool, specs, 1e4, gen, scale=1.0,
                                                          mutate=mutate)
    assert meta.launch.counts.n_wide_items > 0
    seen = 256 + 300 + 130 + prefix + torch.arange(1, new_tokens + 1, dtype=torch.float64)
    a_stored = float(torch.tensor(a, dtype=dtype))
    want = (seen - 1 + torch.tensor(a_stored * (D / 2) / D ** 0.5, dtype=torch.float64).exp()).log()
    got = lse.double().cpu()
    assert torch.allclose(got, want[:, None].expand_as(got), atol=2e-2, rtol=0)
