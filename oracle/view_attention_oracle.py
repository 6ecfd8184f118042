"""CPU oracle for cache-view attention.  TEST INFRASTRUCTURE ONLY.

Nothing under ``async_llm_amd/`` may import this file; only ``tests/``,
``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` use it,
and only as the checker.  It depends on torch (CPU) and numpy alone.

It restates, function by function, what the reference's own code does on this
path.  All citations are relative to ``/root/reference/python/minisgl``:

  apply_rope_correction      shared_cache/rope_correction.py:15-54
  rope_partial               shared_cache/attention.py:241-255
  rope_mrope                 shared_cache/attention.py:130-132, 257-280
  store_kv                   kernel/csrc/jit/store.cu:27-57 (kvcache/mha_pool.py:45-56)
  OBlock / page arithmetic   shared_cache/shared_block.py:24-195
  page_numbers               shared_cache/attention_metadata.py:12-26
  plan_decode                shared_cache/attention.py:282-448
  plan_prefill_batch         shared_cache/attention.py:450-622
  plan_decode_writes         shared_cache/session.py:1102-1141
  forward_decode             shared_cache/attention.py:624-703
  forward_prefill_batch      shared_cache/attention.py:705-752
  get_rope_index             models/qwen3_5_mrope.py:19-64
  copy_shift_kv,             shared_cache/session.py:330-420, 478-528 (merge_blocks, append_block,
  merge_blocks, append_block   _copy_block, _copy_slots, _shift_keys_)

The reference delegates the attention arithmetic itself to FlashInfer 0.6.17
(``pyproject.toml:31``; CUDA only, not vendored, not installable here).  Its
published contract is restated by:

  paged_attention   BatchDecode/BatchPrefillWithPagedKVCacheWrapper.run(return_lse=True):
                    softmax(q K^T / sqrt(D)) V over the first ``seq_len`` tokens of the page
                    list, GQA head h -> kv head h // (Hq/Hkv), optional causal mask aligned to
                    the END of the keys (query i of n sees keys 0 .. kv_len - n + i), output in
                    q's dtype, lse in fp32
  merge_states      flashinfer.merge_states: out = sum_j w_j v_j, w_j = exp(s_j - LSE),
                    LSE = logsumexp_j s_j  (base-invariant for the output)

How each function is pinned (tests/test_oracle_*.py):
  rope functions      closed-form HF neox RoPE, identity at 0, +k/-k round trip, per-dtype
                      tolerances of the reference's test_rope_correction_kernel.py; mRoPE with a
                      scalar position reduces to partial 1-D RoPE; section rule brute-forced
  block arithmetic    known answers of the reference's test_shared_cache.py:51-130
  plan_decode         known answers of test_attention_metadata.py:117-148 and the hand-derived
                      tables of the plumbing configuration (sub_loc 1792/1536/512)
  plan_prefill_batch  known answers of test_attention_metadata.py:151-182
  plan_decode_writes  known answer of test_attention_metadata.py:185-201
  get_rope_index      known answers test_qwen3_5_vision_encoder.py:70-92 and the reference's
                      HF-generated fixtures tests/resources/qwen3_5_0.8B_ref*.npz
  paged_attention,    fp64 brute force per (row, head) on tiny inputs, torch SDPA special case,
  merge_states,       and the global invariant: segment-wise + merge == ONE softmax over the
  forward_*           concatenated view with keys at absolute positions (attention.py:9-16);
                      K=0,V=1 => out == 1 (test_attention_workspace.py:121-125)
  copy_shift_kv,      a merged block read as ONE segment equals the closed-form softmax over
  merge_blocks,       left + right at absolute positions (a wrong sign or amount of the shift fails
  append_block        it); append == merge slot for slot; self-append doubles; shift 0 is a copy
parity unpinned: FlashInfer's internal rounding order and the base (e vs 2) of the LSE it
returns cannot be observed offline; outputs are base-invariant and ``lse_base2`` selects the
convention for the logsumexp.
"""

from __future__ import annotations

import itertools
from dataclasses import dataclass, field
from typing import Dict, List, Optional, Sequence, Tuple

import torch

PAD_LSE = -5.0e4  # zero-weight filler of unused (row, segment) slots (attention.py:697-701)


# ---------------------------------------------------------------------------
# rotation
# ---------------------------------------------------------------------------
def build_cos_sin_cache(rotary_dim: int, max_pos: int, base: float) -> torch.Tensor:
    """``[max_pos, rotary_dim]`` fp32 cos|sin table (layers/rotary.py:24-32,
    shared_cache/session.py:151-161)."""
    inv_freq = 1.0 / (base ** (torch.arange(0, rotary_dim, 2, dtype=torch.float32) / rotary_dim))
    t = torch.arange(max_pos, dtype=torch.float32)
    freqs = torch.einsum("i,j->ij", t, inv_freq)
    return torch.cat((freqs.cos(), freqs.sin()), dim=-1)


def apply_rope_correction(keys: torch.Tensor, corrections: torch.Tensor, cos_sin_cache: torch.Tensor) -> torch.Tensor:
    half = keys.shape[-1] // 2
    idx = corrections.abs().clamp(max=cos_sin_cache.shape[0] - 1)
    cos = cos_sin_cache[idx, :half].unsqueeze(1)
    sin = cos_sin_cache[idx, half:]
    sin = torch.where((corrections < 0).unsqueeze(-1), -sin, sin).unsqueeze(1)
    a = keys[..., :half].to(cos.dtype)
    b = keys[..., half:].to(cos.dtype)
    return torch.cat([cos * a - sin * b, cos * b + sin * a], dim=-1).to(keys.dtype)


def rope_partial(x: torch.Tensor, corrections: torch.Tensor, cos_sin_cache: torch.Tensor, rotary_dim: int) -> torch.Tensor:
    if rotary_dim == x.shape[-1]:
        return apply_rope_correction(x, corrections, cos_sin_cache)
    head = apply_rope_correction(x[..., :rotary_dim].contiguous(), corrections, cos_sin_cache)
    return torch.cat([head, x[..., rotary_dim:]], dim=-1)


def mrope_inv_freq(rotary_dim: int, base: float) -> torch.Tensor:
    return 1.0 / (base ** (torch.arange(0, rotary_dim, 2, dtype=torch.float32) / rotary_dim))


def rope_mrope(x: torch.Tensor, corrections: torch.Tensor, inv_freq: torch.Tensor, mrope_section, rotary_dim: int) -> torch.Tensor:
    pos = corrections.float()
    pos3 = pos if pos.dim() == 2 else pos[None, :].expand(3, -1)
    freqs3 = pos3[:, :, None] * inv_freq[None, None, :]
    freqs = freqs3[0].clone()
    for axis in (1, 2):
        sel = slice(axis, mrope_section[axis] * 3, 3)
        freqs[..., sel] = freqs3[axis][..., sel]
    emb = torch.cat((freqs, freqs), dim=-1)
    cos = emb.cos().to(x.dtype)[:, None, :]
    sin = emb.sin().to(x.dtype)[:, None, :]
    rot, rest = x[..., :rotary_dim], x[..., rotary_dim:]
    h = rot.shape[-1] // 2
    turned = torch.cat((-rot[..., h:], rot[..., :h]), dim=-1)
    return torch.cat([rot * cos + turned * sin, rest], dim=-1)


@dataclass
class RopeSpec:
    """Which rotation a configuration uses."""

    rotary_dim: int
    cos_sin_cache: Optional[torch.Tensor] = None
    mrope_section: Optional[tuple] = None
    inv_freq: Optional[torch.Tensor] = None

    def rotate(self, x: torch.Tensor, pos: torch.Tensor) -> torch.Tensor:
        if self.mrope_section is not None:
            return rope_mrope(x, pos, self.inv_freq, self.mrope_section, self.rotary_dim)
        return rope_partial(x, pos, self.cos_sin_cache, self.rotary_dim)


# ---------------------------------------------------------------------------
# KV store
# ---------------------------------------------------------------------------
def store_kv(k_pool: torch.Tensor, v_pool: torch.Tensor, out_loc: torch.Tensor, k: torch.Tensor, v: torch.Tensor) -> None:
    """Rows with a non-negative slot are copied to ``pool[slot]``; pools are
    ``[num_slots, width]`` views."""
    keep = out_loc >= 0
    slots = out_loc[keep].long()
    k_pool[slots] = k[keep]
    v_pool[slots] = v[keep]


def copy_shift_kv(k_pool: torch.Tensor, v_pool: torch.Tensor, src_slots: Sequence[int], dst_slots: Sequence[int],
                  position_shift: int, rope: "RopeSpec") -> None:
    """One layer of a block copy: rows ``src_slots`` of the ``[num_slots, Hkv, D]``
    pools are gathered and written to ``dst_slots`` (session.py:486-507); then, when
    the destination frame starts ``position_shift`` earlier, the copied keys are
    gathered again, rotated by it as fp32 and written back in the pool's dtype
    (session.py:509-528)."""
    src = torch.as_tensor(src_slots, dtype=torch.int64)
    dst = torch.as_tensor(dst_slots, dtype=torch.int64)
    k_pool.index_copy_(0, dst, k_pool.index_select(0, src))
    v_pool.index_copy_(0, dst, v_pool.index_select(0, src))
    if position_shift:
        corrections = torch.full((dst.numel(),), position_shift, dtype=torch.int64)
        keys = rope.rotate(k_pool.index_select(0, dst).float(), corrections).to(k_pool.dtype)
        k_pool.index_copy_(0, dst, keys)


# ---------------------------------------------------------------------------
# blocks and planners
# ---------------------------------------------------------------------------
@dataclass
class OBlock:
    page_size: int
    page_starts: List[int] = field(default_factory=list)
    num_tokens: int = 0
    mrope_span_override: Optional[int] = None

    @property
    def mrope_span(self) -> int:
        return self.num_tokens if self.mrope_span_override is None else self.mrope_span_override

    @property
    def num_pages(self) -> int:
        return len(self.page_starts)

    @property
    def last_page_len(self) -> int:
        return 0 if self.num_tokens == 0 else self.num_tokens - (self.num_pages - 1) * self.page_size

    @property
    def has_capacity(self) -> bool:
        return self.num_tokens < self.num_pages * self.page_size

    @property
    def free_tail(self) -> int:
        return self.num_pages * self.page_size - self.num_tokens

    def pages_needed(self, n: int) -> int:
        return -(-max(0, n - self.free_tail) // self.page_size)

    def grow_pages(self, starts: Sequence[int], n: int) -> None:
        assert n > 0 and len(starts) == self.pages_needed(n)
        self.page_starts.extend(int(s) for s in starts)
        self.num_tokens += n

    def append_token(self, new_page_start: Optional[int]) -> None:
        if new_page_start is not None:
            assert not self.has_capacity
            self.page_starts.append(int(new_page_start))
        else:
            assert self.has_capacity
        self.num_tokens += 1
        if self.mrope_span_override is not None:
            self.mrope_span_override += 1

    def token_slots(self) -> List[int]:
        return [self.page_starts[i // self.page_size] + i % self.page_size for i in range(self.num_tokens)]


def merge_blocks(layers, left: "OBlock", right: "OBlock", alloc_pages, rope: "RopeSpec") -> "OBlock":
    """``left + right`` in fresh pages (session.py:330-377).  ``layers`` is a list
    of ``(k_pool, v_pool)`` flat ``[num_slots, Hkv, D]`` views, one per layer;
    ``alloc_pages(n)`` returns ``n`` page-start slots."""
    total = left.num_tokens + right.num_tokens
    merged = OBlock(left.page_size)
    merged.page_starts = list(alloc_pages(-(-total // left.page_size)))
    merged.num_tokens = total
    slots = merged.token_slots()
    for k_pool, v_pool in layers:
        if left.num_tokens:
            copy_shift_kv(k_pool, v_pool, left.token_slots(), slots[: left.num_tokens], 0, rope)
        if right.num_tokens:
            copy_shift_kv(k_pool, v_pool, right.token_slots(), slots[left.num_tokens:], left.mrope_span, rope)
    span = left.mrope_span + right.mrope_span
    merged.mrope_span_override = None if span == total else span
    return merged


def append_block(layers, left: "OBlock", right: "OBlock", alloc_pages, rope: "RopeSpec") -> "OBlock":
    """``left += copy of right`` (session.py:379-420); the source layout and both
    spans are taken before ``left`` grows, so ``right is left`` doubles the block."""
    left_tokens, left_span, right_span = left.num_tokens, left.mrope_span, right.mrope_span
    if right.num_tokens:
        source = right.token_slots()
        n = right.num_tokens
        left.grow_pages(list(alloc_pages(left.pages_needed(n))), n)
        target = left.token_slots()[left_tokens: left_tokens + n]
        for k_pool, v_pool in layers:
            copy_shift_kv(k_pool, v_pool, source, target, left_span, rope)
    span = left_span + right_span
    left.mrope_span_override = None if span == left.num_tokens else span
    return left


def page_numbers(block, snapshot: Dict[int, List[int]], extra_page: Optional[int] = None) -> List[int]:
    key = id(block)
    if key not in snapshot:
        pages = [s // block.page_size for s in block.page_starts]
        if extra_page is not None:
            pages.append(extra_page // block.page_size)
        snapshot[key] = pages
    return snapshot[key]


@dataclass
class DecodePlan:
    num_workers: int
    max_segments: int
    n_main: int
    n_aux: int
    sub_worker: List[int]
    sub_loc: List[int]
    pad_slot: List[int]
    kv_indptr: List[int]
    kv_indices: List[int]
    seq_lens: List[int]
    last_page_len: List[int]
    aux_slots: List[int]


def plan_decode(views, write_to, new_page_for_block: Dict[int, Optional[int]], new_token_slots: Sequence[int],
                page_size: int) -> DecodePlan:
    write_set = set(new_page_for_block)
    snap: Dict[int, List[int]] = {}
    mw, ml, ms, parts, lens, last = [], [], [], [], [], []
    aw, al, asl, akv = [], [], [], []
    max_segments = 0
    for w, (view, wt) in enumerate(zip(views, write_to)):
        lengths = [b.num_tokens + (1 if id(b) in write_set else 0) for b in view]
        spans = [b.mrope_span + (1 if id(b) in write_set else 0) for b in view]
        total = sum(spans)
        n_seg = 0
        prefix = 0
        for b, length, span in zip(view, lengths, spans):
            if length == 0:
                prefix += span
                continue
            pages = page_numbers(b, snap, new_page_for_block.get(id(b)))
            mw.append(w)
            ml.append(total - prefix - 1)
            ms.append(n_seg)
            parts.append(pages)
            lens.append(length)
            last.append(length - (len(pages) - 1) * page_size)
            n_seg += 1
            prefix += span
        if not any(b is wt for b in view):
            aw.append(w)
            al.append(wt.mrope_span)
            asl.append(n_seg)
            akv.append(int(new_token_slots[w]))
            n_seg += 1
        max_segments = max(max_segments, n_seg)
    sub_worker = mw + aw
    slots = ms + asl
    indptr = [0]
    for p in parts:
        indptr.append(indptr[-1] + len(p))
    return DecodePlan(
        num_workers=len(views), max_segments=max_segments, n_main=len(mw), n_aux=len(aw),
        sub_worker=sub_worker, sub_loc=ml + al,
        pad_slot=[w * max_segments + s for w, s in zip(sub_worker, slots)],
        kv_indptr=indptr, kv_indices=[p for part in parts for p in part], seq_lens=lens,
        last_page_len=last, aux_slots=akv)


@dataclass
class OPrefillSpec:
    context: List[OBlock]
    self_page_starts: List[int]
    num_new: int
    self_prefix_len: int = 0
    self_prefix_span: Optional[int] = None
    mrope_rel: Optional[torch.Tensor] = None  # [3, num_new] int64


@dataclass
class PrefillPlan:
    num_rows: int
    max_segments: int
    n_ctx_rows: int
    sub_worker: List[int]
    sub_loc: torch.Tensor  # [N] or [3, N] int64
    pad_slot: List[int]
    last_indices: List[int]
    ctx: dict
    own: dict


def plan_prefill_batch(specs: Sequence[OPrefillSpec], page_size: int) -> PrefillPlan:
    assert specs
    use_3d = any(s.mrope_rel is not None for s in specs)
    M = max(len(s.context) + 1 for s in specs)
    snap: Dict[int, List[int]] = {}
    cg, cs, cl, cparts, cq, clen, clast = [], [], [], [], [], [], []
    sg, ss, sl, sparts, sq, slen, slast = [], [], [], [], [], [], []
    last_indices = []
    offset = 0

    def rel_positions(spec):
        if spec.mrope_rel is None:
            r = torch.arange(spec.num_new, dtype=torch.int64)
            return r.view(1, -1).expand(3, -1) if use_3d else r
        r = spec.mrope_rel.to(torch.int64)
        assert r.shape == (3, spec.num_new)
        return r

    for spec in specs:
        S, T = int(spec.num_new), int(spec.self_prefix_len)
        assert S > 0
        T_span = T if spec.self_prefix_span is None else int(spec.self_prefix_span)
        spans = [b.mrope_span for b in spec.context]
        self_offset = sum(spans) + T_span
        rows = list(range(offset, offset + S))
        rel = rel_positions(spec)
        prefix = 0
        for j, (b, span) in enumerate(zip(spec.context, spans)):
            assert b.num_tokens > 0
            cg.extend(rows)
            cs.extend([j] * S)
            cl.append(rel + (self_offset - prefix))
            cparts.append(page_numbers(b, snap))
            cq.append(S)
            clen.append(b.num_tokens)
            clast.append(b.last_page_len)
            prefix += span
        pages = [s // page_size for s in spec.self_page_starts]
        sg.extend(rows)
        ss.extend([len(spec.context)] * S)
        sl.append(rel + T_span)
        sparts.append(pages)
        sq.append(S)
        slen.append(T + S)
        slast.append(T + S - (len(pages) - 1) * page_size)
        last_indices.append(offset + S - 1)
        offset += S

    def table(parts, qlens, lens, lasts, causal):
        indptr, qo = [0], [0]
        for p in parts:
            indptr.append(indptr[-1] + len(p))
        for n in qlens:
            qo.append(qo[-1] + n)
        return dict(qo_indptr=qo, kv_indptr=indptr, kv_indices=[p for part in parts for p in part],
                    seq_lens=lens, last_page_len=lasts, causal=causal,
                    max_token_per_sequence=max(qlens) if qlens else 0)

    gather = cg + sg
    slot = cs + ss
    return PrefillPlan(
        num_rows=offset, max_segments=M, n_ctx_rows=len(cg), sub_worker=gather,
        sub_loc=torch.cat(cl + sl, dim=1 if use_3d else 0),
        pad_slot=[r * M + s for r, s in zip(gather, slot)], last_indices=last_indices,
        ctx=table(cparts, cq, clen, clast, False), own=table(sparts, sq, slen, slast, True))


def plan_decode_writes(write_to: Sequence[OBlock], page_size: int, alloc_pages) -> Tuple[Dict[int, Optional[int]], List[int], List[int]]:
    """Destination slot of each writer's new token; one bulk page allocation for
    all writers whose last page is full.  ``alloc_pages(n)`` returns ``n``
    page-start slots."""
    pending: Dict[int, Optional[int]] = {}
    need = []
    for wt in write_to:
        if id(wt) in pending:
            raise ValueError("WorkerGroup has two workers writing the same block in one step")
        pending[id(wt)] = None
        if not wt.has_capacity:
            need.append(wt)
    if need:
        for wt, start in zip(need, [int(s) for s in alloc_pages(len(need))]):
            pending[id(wt)] = start
    out_loc, write_pos = [], []
    for wt in write_to:
        new_page = pending[id(wt)]
        page_start = new_page if new_page is not None else wt.page_starts[-1]
        out_loc.append(page_start + wt.num_tokens % page_size)
        write_pos.append(wt.mrope_span)
    return pending, out_loc, write_pos


# ---------------------------------------------------------------------------
# mRoPE positions
# ---------------------------------------------------------------------------
def vision_position_ids_3d(start: int, t: int, h: int, w: int, merge: int) -> torch.Tensor:
    lt, lh, lw = t, h // merge, w // merge
    pt = torch.arange(lt).repeat_interleave(lh * lw) + start
    ph = (torch.arange(lh) + start).repeat_interleave(lw).repeat(lt)
    pw = (torch.arange(lw) + start).repeat(lh * lt)
    return torch.stack([pt, ph, pw], dim=0)


def get_rope_index(mm_token_type_ids: Sequence[int], spatial_merge_size: int, image_grid_thw=None) -> torch.Tensor:
    grids = iter(image_grid_thw if image_grid_thw is not None else ())
    parts, cur = [], 0
    for key, run in itertools.groupby(mm_token_type_ids):
        n = len(list(run))
        if key == 0:
            parts.append(torch.arange(n).view(1, -1).expand(3, -1) + cur)
            cur += n
        elif key in (1, 2):
            t, h, w = (int(v) for v in next(grids))
            parts.append(vision_position_ids_3d(cur, t, h, w, spatial_merge_size))
            cur += max(h, w) // spatial_merge_size
        else:
            raise NotImplementedError(key)
    return torch.cat(parts, dim=1).reshape(3, -1)


# ---------------------------------------------------------------------------
# attention arithmetic
# ---------------------------------------------------------------------------
def gather_tokens(paged: torch.Tensor, pages: Sequence[int], seq_len: int) -> torch.Tensor:
    """First ``seq_len`` token rows ``[seq_len, Hkv, D]`` of a page list over
    ``paged [num_pages, page_size, Hkv, D]``."""
    idx = torch.as_tensor(pages, dtype=torch.long)
    return paged[idx].reshape(-1, paged.shape[-2], paged.shape[-1])[:seq_len]


def paged_attention(q: torch.Tensor, keys: torch.Tensor, values: torch.Tensor, causal: bool = False,
                    math_dtype: torch.dtype = torch.float32, out_dtype: Optional[torch.dtype] = None):
    """``q [n, Hq, D]`` against ``keys/values [L, Hkv, D]``.  Returns ``out [n,
    Hq, D]`` in ``out_dtype`` (default q's) and natural-log ``lse [n, Hq]`` in
    ``math_dtype``.  Causal: query i sees keys ``0 .. L - n + i``."""
    n, Hq, D = q.shape
    L, Hkv, _ = keys.shape
    g = Hq // Hkv
    qf = q.to(math_dtype).view(n, Hkv, g, D)
    kf = keys.to(math_dtype)
    vf = values.to(math_dtype)
    s = torch.einsum("nkgd,lkd->nkgl", qf, kf) / (D ** 0.5)
    if causal:
        visible = torch.arange(L)[None, :] <= (L - n + torch.arange(n))[:, None]
        s = s.masked_fill(~visible[:, None, None, :], float("-inf"))
    lse = torch.logsumexp(s, dim=-1)
    p = torch.exp(s - lse.unsqueeze(-1))
    o = torch.einsum("nkgl,lkd->nkgd", p, vf).reshape(n, Hq, D)
    return o.to(out_dtype or q.dtype), lse.reshape(n, Hq)


def merge_states(v: torch.Tensor, s: torch.Tensor):
    """``v [W, M, H, D]``, ``s [W, M, H]`` (logsumexp per state, any one base as
    long as ``exp`` below matches: natural here).  Returns merged ``[W, H, D]``
    in v's dtype and ``[W, H]`` fp32/fp64."""
    sf = s.to(torch.float64 if s.dtype == torch.float64 else torch.float32)
    top = sf.max(dim=1, keepdim=True).values
    w = torch.exp(sf - top)
    denom = w.sum(dim=1)
    merged = (v.to(sf.dtype) * w.unsqueeze(-1)).sum(dim=1) / denom.unsqueeze(-1)
    return merged.to(v.dtype), (top.squeeze(1) + torch.log(denom))


def _pad_merge(out: torch.Tensor, lse: torch.Tensor, pad_slot: Sequence[int], rows: int, M: int):
    Hq, D = out.shape[1], out.shape[2]
    v_pad = out.new_zeros(rows * M, Hq, D)
    s_pad = torch.full((rows * M, Hq), PAD_LSE, dtype=lse.dtype)
    slot = torch.as_tensor(pad_slot, dtype=torch.long)
    v_pad[slot] = out
    s_pad[slot] = lse
    return merge_states(v_pad.view(rows, M, Hq, D), s_pad.view(rows, M, Hq))


def forward_decode(plan: DecodePlan, q: torch.Tensor, k_paged: torch.Tensor, v_paged: torch.Tensor, rope: RopeSpec,
                   math_dtype: torch.dtype = torch.float32):
    """Decode attention AFTER the new K/V rows were stored.  ``q [W, Hq, D]``
    unrotated.  Returns merged ``out [W, Hq*D]`` (q's dtype), merged natural-log
    ``lse [W, Hq]`` and the per-sub-request ``(out, lse)`` lists."""
    W, Hq, D = q.shape
    q_sub = rope.rotate(q[torch.as_tensor(plan.sub_worker, dtype=torch.long)],
                        torch.as_tensor(plan.sub_loc, dtype=torch.int64))
    outs, lses = [], []
    for i in range(plan.n_main):
        pages = plan.kv_indices[plan.kv_indptr[i]:plan.kv_indptr[i + 1]]
        keys = gather_tokens(k_paged, pages, plan.seq_lens[i])
        vals = gather_tokens(v_paged, pages, plan.seq_lens[i])
        o, l = paged_attention(q_sub[i:i + 1], keys, vals, math_dtype=math_dtype)
        outs.append(o)
        lses.append(l)
    kflat = k_paged.reshape(-1, k_paged.shape[-2], k_paged.shape[-1])
    vflat = v_paged.reshape(-1, v_paged.shape[-2], v_paged.shape[-1])
    for j, slot in enumerate(plan.aux_slots):
        i = plan.n_main + j
        o, l = paged_attention(q_sub[i:i + 1], kflat[slot:slot + 1], vflat[slot:slot + 1], math_dtype=math_dtype)
        outs.append(o)
        lses.append(l)
    out = torch.cat(outs, dim=0)
    lse = torch.cat(lses, dim=0)
    if plan.max_segments == 1 and plan.n_aux == 0:
        return out.reshape(W, -1), lse, (outs, lses)
    merged, mlse = _pad_merge(out, lse, plan.pad_slot, W, plan.max_segments)
    return merged.reshape(W, -1), mlse, (outs, lses)


def forward_prefill_batch(plan: PrefillPlan, q: torch.Tensor, k_paged: torch.Tensor, v_paged: torch.Tensor,
                          rope: RopeSpec, math_dtype: torch.dtype = torch.float32):
    """Prefill attention AFTER the new K/V rows were stored.  ``q [N, Hq, D]``
    unrotated, request-major."""
    N, Hq, D = q.shape
    q_sub = rope.rotate(q[torch.as_tensor(plan.sub_worker, dtype=torch.long)], plan.sub_loc)

    def run(tab, base):
        outs, lses = [], []
        for i in range(len(tab["seq_lens"])):
            rows = slice(base + tab["qo_indptr"][i], base + tab["qo_indptr"][i + 1])
            pages = tab["kv_indices"][tab["kv_indptr"][i]:tab["kv_indptr"][i + 1]]
            keys = gather_tokens(k_paged, pages, tab["seq_lens"][i])
            vals = gather_tokens(v_paged, pages, tab["seq_lens"][i])
            o, l = paged_attention(q_sub[rows], keys, vals, causal=tab["causal"], math_dtype=math_dtype)
            outs.append(o)
            lses.append(l)
        return outs, lses

    so, sl = run(plan.own, plan.n_ctx_rows)
    if plan.n_ctx_rows == 0:
        return torch.cat(so, dim=0).reshape(N, -1), torch.cat(sl, dim=0)
    co, cl = run(plan.ctx, 0)
    out = torch.cat(co + so, dim=0)
    lse = torch.cat(cl + sl, dim=0)
    merged, mlse = _pad_merge(out, lse, plan.pad_slot, N, plan.max_segments)
    return merged.reshape(N, -1), mlse


# ---------------------------------------------------------------------------
# independent closed form: one softmax over the concatenated view
# ---------------------------------------------------------------------------
def concat_view_attention(q_row: torch.Tensor, q_pos: int, raw_keys: Sequence[torch.Tensor], values: Sequence[torch.Tensor],
                          starts: Sequence[int], rel_pos: Sequence[torch.Tensor], rotary_dim: int, base: float):
    """fp64 attention of one unrotated query ``q_row [Hq, D]`` at absolute
    position ``q_pos`` over segments of UNROTATED keys ``raw_keys[j] [L_j, Hkv, D]``
    whose token i sits at absolute position ``starts[j] + rel_pos[j][i]``; plain
    1-D RoPE computed in fp64 from its definition.  Returns ``out [Hq, D]`` and
    natural-log ``lse [Hq]``."""
    def rot(x, pos):
        x = x.double()
        half = rotary_dim // 2
        inv = 1.0 / (torch.tensor(base, dtype=torch.float64) ** (torch.arange(0, rotary_dim, 2, dtype=torch.float64) / rotary_dim))
        ang = pos.double()[:, None] * inv[None, :]
        c, s = ang.cos()[:, None, :], ang.sin()[:, None, :]
        a, b = x[..., :half], x[..., half:rotary_dim]
        return torch.cat([a * c - b * s, b * c + a * s, x[..., rotary_dim:]], dim=-1)

    Hq, D = q_row.shape
    qr = rot(q_row[None], torch.tensor([q_pos]))[0]
    ks = torch.cat([rot(k, torch.as_tensor(r) + st) for k, st, r in zip(raw_keys, starts, rel_pos)], dim=0)
    vs = torch.cat([v.double() for v in values], dim=0)
    Hkv = ks.shape[1]
    g = Hq // Hkv
    s = torch.einsum("kgd,lkd->kgl", qr.view(Hkv, g, D), ks) / (D ** 0.5)
    lse = torch.logsumexp(s, dim=-1)
    o = torch.einsum("kgl,lkd->kgd", torch.exp(s - lse[..., None]), vs)
    return o.reshape(Hq, D), lse.reshape(Hq)
