"""Seeded synthetic view-attention workloads: the five benchmark configurations
and scaled-down versions of them for tests.

Every builder returns a :class:`Workload`: the op, a paged pool with several
layers (distinct HBM copies to rotate over while timing), the blocks and views,
the planned metadata, unrotated q/k/v for one step and the byte / flop
accounting of one ``forward``.

Accounting (per forward, one layer):
  * ``alg_bytes``: compulsory HBM traffic.  K and V of every DISTINCT block a
    launch references count once (``2*Hkv*D*itemsize`` per token, lengths taken
    after this step's appends), plus q in and out, the lse, the int32 index
    tables, and the new rows stored into the pool.
  * ``logical_bytes``: K and V counted once per (row, segment) -- what a
    per-sub-request execution reads.
  * ``alg_flops``: ``4*D*Hq`` per visible (query row, key) pair.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from types import SimpleNamespace
from typing import Dict, List, Optional

import torch

from .kvcache import MHAKVCache
from .shared_cache import CacheBlock, PrefillSpec, SharedCacheAttention, WorkerGroup
from .shared_cache.mrope import get_rope_index
from .shared_cache.session_planning import plan_decode_writes


@dataclass
class Workload:
    name: str
    mode: str  # "decode" | "prefill"
    op: SharedCacheAttention
    pool: MHAKVCache
    q: torch.Tensor
    k: torch.Tensor
    v: torch.Tensor
    batch: SimpleNamespace
    blocks: List[CacheBlock]
    theta: float
    group: Optional[WorkerGroup] = None
    pending: Optional[Dict[int, Optional[int]]] = None
    new_token_slots: Optional[torch.Tensor] = None
    specs: Optional[List[PrefillSpec]] = None
    alg_bytes: int = 0
    logical_bytes: int = 0
    alg_flops: int = 0
    info: dict = field(default_factory=dict)

    @property
    def meta(self):
        return self.batch.attn_metadata

    def forward(self, layer: int = 0) -> torch.Tensor:
        return self.op.forward(self.q, self.k, self.v, layer, self.batch)


class _Pages:
    """Hands out the pages of a seeded random permutation, in order."""

    def __init__(self, num_pages: int, page_size: int, gen: torch.Generator):
        self.order = torch.randperm(num_pages, generator=gen).tolist()
        self.page_size = page_size
        self.used = 0

    def take(self, n: int) -> List[int]:
        assert self.used + n <= len(self.order), "pool too small for this workload"
        got = self.order[self.used:self.used + n]
        self.used += n
        return [p * self.page_size for p in got]

    # PageAllocator-shaped access for plan_decode_writes
    def alloc_pages(self, n: int) -> torch.Tensor:
        return torch.tensor(self.take(n), dtype=torch.int32)


def _filled_block(pages: _Pages, device, page_size: int, length: int, span: Optional[int] = None) -> CacheBlock:
    b = CacheBlock(device, page_size)
    if length:
        starts = pages.take(-(-length // page_size))
        b.grow_pages(torch.tensor(starts, dtype=torch.int32), length)
    if span is not None:
        b.mrope_span_override = span
    return b


def build_cos_sin_cache(rotary_dim: int, max_pos: int, base: float, device) -> torch.Tensor:
    """fp32 ``[max_pos, rotary_dim]`` cos|sin table in the format of the reference
    (``layers/rotary.py:24-32``)."""
    inv_freq = 1.0 / (base ** (torch.arange(0, rotary_dim, 2, dtype=torch.float32) / rotary_dim))
    t = torch.arange(max_pos, dtype=torch.float32)
    freqs = torch.einsum("i,j->ij", t, inv_freq)
    return torch.cat((freqs.cos(), freqs.sin()), dim=-1).to(device)


def _make_pool(hkv, d, num_pages, page, dtype, device, layers, seed, scale):
    pool = MHAKVCache(hkv, layers, d, num_pages, page, dtype, device)
    gen = torch.Generator(device=device).manual_seed(seed)
    for layer in range(layers):
        _fill_normal(pool.k_cache(layer), gen, scale)
        _fill_normal(pool.v_cache(layer), gen, scale)
    return pool


def _fill_normal(cache: torch.Tensor, gen: torch.Generator, scale: float) -> None:
    """N(0, scale^2) fill in page chunks, so the fp32 staging stays small."""
    step = max(1, (1 << 26) // cache[0].numel())
    for a in range(0, cache.shape[0], step):
        part = cache[a:a + step]
        noise = torch.randn(part.shape, generator=gen, device=cache.device, dtype=torch.float32)
        part.copy_((noise * scale).to(cache.dtype))


def _decode_accounting(op: SharedCacheAttention, group: WorkerGroup, pending, meta, itemsize: int):
    b_tok = 2 * op.num_kv_heads * op.head_dim * itemsize
    W = group.num_workers
    written = set(pending)
    distinct: Dict[int, int] = {}
    logical = 0
    for view, target in zip(group.cache_structure, group.write_to):
        for b in view:
            n = b.num_tokens + (1 if id(b) in written else 0)
            distinct[id(b)] = n
            logical += n
        if not any(b is target for b in view):
            distinct.setdefault(id(target), target.num_tokens + 1)
            logical += 1
    unique = sum(distinct.values())
    n_sub = meta.n_main + meta.n_aux
    tables = meta.launch.kv_indices.numel() + 2 * n_sub + 1
    alg = (b_tok * unique + 2 * W * op.num_qo_heads * op.head_dim * itemsize + 4 * W * op.num_qo_heads
           + 4 * tables + W * b_tok)
    return alg, b_tok * logical, 4 * op.head_dim * op.num_qo_heads * logical


def _finish_decode(name, op, pool, blocks, views, write_to, pages, device, dtype, gen, theta, scale_qkv,
                   mrope_positions=None) -> Workload:
    group = WorkerGroup(cache_structure=views, write_to=write_to)
    pending, slots, write_pos = plan_decode_writes(group, op.page_size, pages, device)
    meta = op.prepare(group, pending, slots)
    W = group.num_workers
    Hq, Hkv, D = op.num_qo_heads, op.num_kv_heads, op.head_dim
    q = (torch.randn(W, Hq * D, generator=gen) * scale_qkv).to(dtype).to(device)
    k = (torch.randn(W, Hkv * D, generator=gen) * scale_qkv).to(dtype).to(device)
    v = (torch.randn(W, Hkv * D, generator=gen) * scale_qkv).to(dtype).to(device)
    batch = SimpleNamespace(attn_metadata=meta, positions=torch.tensor(write_pos, dtype=torch.int64, device=device),
                            out_loc=slots, mrope_positions=mrope_positions)
    alg, logical, flops = _decode_accounting(op, group, pending, meta, q.element_size())
    return Workload(name, "decode", op, pool, q, k, v, batch, blocks, theta, group=group, pending=pending,
                    new_token_slots=slots, alg_bytes=alg, logical_bytes=logical, alg_flops=flops,
                    info=dict(rows=W, sub_requests=meta.n_main + meta.n_aux))


def plumbing_decode(device, layers: int = 1, kernel: Optional[str] = None) -> Workload:
    """Configuration 1: fp32, one worker over a 3-block view 256/1024/512 (P 16,
    256-page pool), 8 q / 2 kv heads, head_dim 128, theta 1e6, seed 0."""
    dtype, Hq, Hkv, D, P, theta = torch.float32, 8, 2, 128, 16, 1e6
    gen = torch.Generator().manual_seed(0)
    pages = _Pages(256, P, gen)
    pool = _make_pool(Hkv, D, 256, P, dtype, device, layers, 0, D ** -0.5)
    table = build_cos_sin_cache(D, 4096, theta, device)
    op = SharedCacheAttention(pool, table, Hq, Hkv, D, P, dtype, device, kernel=kernel)
    blocks = [_filled_block(pages, device, P, n) for n in (256, 1024, 512)]
    return _finish_decode("plumbing_decode", op, pool, blocks, [blocks], [blocks[2]], pages, device, dtype, gen,
                          theta, D ** -0.5)


def batched_decode(device, workers: int = 64, shared_len: int = 8192, private_lo: int = 256,
                   private_hi: int = 8192, layers: int = 1, rotary_dim: Optional[int] = None,
                   heads=(16, 4, 256), dtype=torch.bfloat16, page_size: int = 16, seed: int = 1,
                   kernel: Optional[str] = None) -> Workload:
    """Configuration 2: every view is one shared prompt block followed by 1-3
    private blocks with lengths uniform in [private_lo, private_hi]; each
    worker appends to its last private block; theta 1e7."""
    Hq, Hkv, D = heads
    P, theta = page_size, 1e7
    gen = torch.Generator().manual_seed(seed)
    counts = torch.randint(1, 4, (workers,), generator=gen).tolist()
    lengths = [torch.randint(private_lo, private_hi + 1, (c,), generator=gen).tolist() for c in counts]
    need = -(-shared_len // P) + sum(-(-n // P) + 1 for ls in lengths for n in ls) + workers
    pages = _Pages(need, P, gen)
    pool = _make_pool(Hkv, D, need, P, dtype, device, layers, seed, 1.0)
    rd = D if rotary_dim is None else rotary_dim
    max_pos = shared_len + 3 * private_hi + 64
    op = SharedCacheAttention(pool, build_cos_sin_cache(rd, max_pos, theta, device), Hq, Hkv, D, P, dtype, device,
                              rotary_dim=rd, kernel=kernel)
    shared = _filled_block(pages, device, P, shared_len)
    blocks, views, write_to = [shared], [], []
    for ls in lengths:
        private = [_filled_block(pages, device, P, n) for n in ls]
        blocks += private
        views.append([shared] + private)
        write_to.append(private[-1])
    return _finish_decode("batched_decode", op, pool, blocks, views, write_to, pages, device, dtype, gen, theta, 1.0)


def mrope_decode(device, workers: int = 8, blocks_per_view: int = 8, block_len: int = 16384,
                 image_tokens: int = 4096, layers: int = 1, heads=(16, 4, 256), dtype=torch.bfloat16,
                 page_size: int = 16, seed: int = 4, kernel: Optional[str] = None) -> Workload:
    """Configuration 5: long-context decode with interleaved mRoPE (sections
    24/20/20 of 64 rotary pairs, theta 1e7).  Every block holds an image span of
    ``image_tokens`` tokens laid out on a square grid, which advances the running
    position by the grid side only, so the block's span is
    ``block_len - image_tokens + side``."""
    Hq, Hkv, D = heads
    P, theta = page_size, 1e7
    rd, section = 128 if D >= 128 else D, (24, 20, 20) if D >= 128 else (D // 2 - 2 * (D // 8), D // 8, D // 8)
    side = int(round(image_tokens ** 0.5))
    assert side * side == image_tokens
    # a block's tokens: text, one image of side x side merged patches (grid 1 x 2 side x 2 side at
    # merge size 2), text; its span is one past the last position get_rope_index gives them
    lead = (block_len - image_tokens) // 4
    kinds = torch.tensor([0] * lead + [1] * image_tokens + [0] * (block_len - image_tokens - lead))
    block_positions = get_rope_index(kinds, kinds, 2, torch.tensor([[1, 2 * side, 2 * side]]))
    span = int(block_positions.max()) + 1
    assert span == block_len - image_tokens + side
    gen = torch.Generator().manual_seed(seed)
    need = workers * blocks_per_view * (-(-block_len // P) + 1)
    pages = _Pages(need, P, gen)
    pool = _make_pool(Hkv, D, need, P, dtype, device, layers, seed, 1.0)
    op = SharedCacheAttention(pool, torch.zeros(1, rd, device=device), Hq, Hkv, D, P, dtype, device, rotary_dim=rd,
                              mrope_section=section, rope_base=theta, kernel=kernel)
    blocks, views, write_to = [], [], []
    for _ in range(workers):
        mine = [_filled_block(pages, device, P, block_len, span) for _ in range(blocks_per_view)]
        blocks += mine
        views.append(mine)
        write_to.append(mine[-1])
    wl = _finish_decode("mrope_decode", op, pool, blocks, views, write_to, pages, device, dtype, gen, theta, 1.0)
    wl.info.update(mrope_section=section, block_span=span)
    return wl


def view_prefill(device, requests: int = 8, new_tokens: int = 2048, own_prefix: int = 1024,
                 prompt_len: int = 32768, layers: int = 1, heads=(16, 4, 256), dtype=torch.bfloat16,
                 page_size: int = 16, seed: int = 2, rotary_dim: Optional[int] = None,
                 kernel: Optional[str] = None) -> Workload:
    """Configuration 3: every request extends its own block (``own_prefix``
    tokens) by ``new_tokens`` and attends to a shared prompt block plus the other
    requests' blocks at their pre-write length."""
    Hq, Hkv, D = heads
    P, theta = page_size, 1e7
    gen = torch.Generator().manual_seed(seed)
    need = -(-prompt_len // P) + requests * (-(-(own_prefix + new_tokens) // P) + 1)
    pages = _Pages(need, P, gen)
    pool = _make_pool(Hkv, D, need, P, dtype, device, layers, seed, 1.0)
    rd = D if rotary_dim is None else rotary_dim
    max_pos = prompt_len + requests * own_prefix + new_tokens + 64
    op = SharedCacheAttention(pool, build_cos_sin_cache(rd, max_pos, theta, device), Hq, Hkv, D, P, dtype, device,
                              rotary_dim=rd, kernel=kernel)
    prompt = _filled_block(pages, device, P, prompt_len)
    own = [_filled_block(pages, device, P, own_prefix) for _ in range(requests)]
    specs, positions, out_loc = [], [], []
    pairs = 0
    for r, block in enumerate(own):
        fresh = pages.take(block.pages_needed(new_tokens))
        all_starts = torch.tensor(block.page_starts + fresh, dtype=torch.int32)
        context = [b for b in [prompt] + [o for i, o in enumerate(own) if i != r] if b.num_tokens > 0]
        specs.append(PrefillSpec(context, all_starts, new_tokens, own_prefix))
        slots = (all_starts[:, None] + torch.arange(P, dtype=torch.int32)[None, :]).reshape(-1)
        out_loc.append(slots[own_prefix:own_prefix + new_tokens])
        positions.append(torch.arange(own_prefix, own_prefix + new_tokens, dtype=torch.int64))
        pairs += new_tokens * sum(b.num_tokens for b in context) + new_tokens * own_prefix + new_tokens * (new_tokens + 1) // 2
    meta = op.prepare_prefill_batch(specs)
    N = requests * new_tokens
    q = torch.randn(N, Hq * D, generator=gen).to(dtype).to(device)
    k = torch.randn(N, Hkv * D, generator=gen).to(dtype).to(device)
    v = torch.randn(N, Hkv * D, generator=gen).to(dtype).to(device)
    batch = SimpleNamespace(attn_metadata=meta, positions=torch.cat(positions).to(device),
                            out_loc=torch.cat(out_loc).to(device), mrope_positions=None)
    item = q.element_size()
    b_tok = 2 * Hkv * D * item
    distinct = prompt.num_tokens + requests * (own_prefix + new_tokens)
    alg_bytes = b_tok * distinct + 2 * N * Hq * D * item + N * b_tok
    return Workload("view_prefill", "prefill", op, pool, q, k, v, batch, [prompt] + own, theta, specs=specs,
                    alg_bytes=alg_bytes, logical_bytes=b_tok * pairs // max(1, new_tokens),
                    alg_flops=4 * D * Hq * pairs, info=dict(rows=N, visible_pairs=pairs))


def mixed_batch(device, decode_rows: int = 48, chunks: int = 4, chunk_len: int = 512, ctx_lo: int = 1024,
                ctx_hi: int = 32768, shared_len: int = 512, layers: int = 1, heads=(16, 4, 256),
                dtype=torch.bfloat16, page_size: int = 16, seed: int = 3, kernel: Optional[str] = None) -> Workload:
    """Configuration 4: a continuous batch in ONE launch -- ``decode_rows`` decode
    requests plus ``chunks`` prefill chunks of ``chunk_len`` tokens.  Every view
    starts with the shared prompt block and has 2-5 blocks in total; the total
    context per row is uniform in [ctx_lo, ctx_hi] and split over the private
    blocks by a seeded random composition (every block >= 16 tokens).  Decode rows
    append to their last block; a chunk row extends its last block (the block's
    current length is the chunk's prefix) and reads the blocks before it."""
    Hq, Hkv, D = heads
    P, theta = page_size, 1e7
    gen = torch.Generator().manual_seed(seed)
    rows = decode_rows + chunks
    totals = torch.randint(ctx_lo, ctx_hi + 1, (rows,), generator=gen).tolist()
    counts = torch.randint(2, 6, (rows,), generator=gen).tolist()
    splits = []
    for total, n in zip(totals, counts):
        rest, parts = max(total - shared_len, 16 * (n - 1)), n - 1
        w = torch.rand(parts, generator=gen)
        extra = ((rest - 16 * parts) * w / w.sum()).floor().to(torch.int64).tolist()
        lens = [16 + e for e in extra]
        lens[-1] += rest - sum(lens)
        splits.append(lens)
    need = -(-shared_len // P) + sum(-(-n // P) + 1 for ls in splits for n in ls) + chunks * (chunk_len // P + 2) + rows
    pages = _Pages(need, P, gen)
    pool = _make_pool(Hkv, D, need, P, dtype, device, layers, seed, 1.0)
    op = SharedCacheAttention(pool, build_cos_sin_cache(D, ctx_hi + chunk_len + shared_len + 64, theta, device), Hq, Hkv, D,
                              P, dtype, device, kernel=kernel)
    shared = _filled_block(pages, device, P, shared_len)
    blocks, views, write_to, specs = [shared], [], [], []
    positions, out_loc = [], []
    pairs = 0
    for r, ls in enumerate(splits):
        mine = [_filled_block(pages, device, P, n) for n in ls]
        blocks += mine
        if r < decode_rows:
            views.append([shared] + mine)
            write_to.append(mine[-1])
        else:
            own, context = mine[-1], [shared] + mine[:-1]
            fresh = pages.take(own.pages_needed(chunk_len))
            starts = torch.tensor(own.page_starts + fresh, dtype=torch.int32)
            specs.append(PrefillSpec(context, starts, chunk_len, own.num_tokens))
            slots = (starts[:, None] + torch.arange(P, dtype=torch.int32)[None, :]).reshape(-1)
            out_loc.append(slots[own.num_tokens:own.num_tokens + chunk_len])
            positions.append(torch.arange(own.num_tokens, own.num_tokens + chunk_len, dtype=torch.int64))
            pairs += chunk_len * (sum(b.num_tokens for b in context) + own.num_tokens) + chunk_len * (chunk_len + 1) // 2
    group = WorkerGroup(cache_structure=views, write_to=write_to)
    pending, slots_d, write_pos = plan_decode_writes(group, P, pages, device)
    meta = op.prepare_mixed(group, pending, slots_d, specs)
    N = decode_rows + chunks * chunk_len
    q = torch.randn(N, Hq * D, generator=gen).to(dtype).to(device)
    k = torch.randn(N, Hkv * D, generator=gen).to(dtype).to(device)
    v = torch.randn(N, Hkv * D, generator=gen).to(dtype).to(device)
    batch = SimpleNamespace(
        attn_metadata=meta,
        positions=torch.cat([torch.tensor(write_pos, dtype=torch.int64)] + positions).to(device),
        out_loc=torch.cat([slots_d.cpu()] + out_loc).to(device), mrope_positions=None)
    item = q.element_size()
    b_tok = 2 * Hkv * D * item
    distinct = sum(b.num_tokens for b in blocks) + decode_rows + chunks * chunk_len
    logical = sum(sum(b.num_tokens for b in view) + 1 for view in views)
    alg_bytes = b_tok * distinct + 2 * N * Hq * D * item + 4 * N * Hq + 4 * meta.launch.kv_indices.numel() + N * b_tok
    return Workload("mixed_batch", "mixed", op, pool, q, k, v, batch, blocks, theta, group=group, pending=pending,
                    new_token_slots=slots_d, specs=specs, alg_bytes=alg_bytes, logical_bytes=b_tok * logical,
                    alg_flops=4 * D * Hq * (pairs + logical),
                    info=dict(rows=N, decode_rows=decode_rows, chunks=chunks, chunk_len=chunk_len,
                              prefill_pairs=pairs))
