"""Cache-view attention on MI355X: one request attends to an ordered list of
shared, paged ``CacheBlock`` s.

Drop-in for the reference ``SharedCacheAttention`` / ``SharedCacheAttnMetadata``
/ ``PrefillSpec`` (``python/minisgl/shared_cache/attention.py``): same
constructor, ``prepare`` / ``prepare_prefill_batch`` / ``forward`` /
``prepare_workspace`` signatures, same metadata fields, same integer tables.
What differs is everything below the tables.  The reference rotates and copies
one query per (row, segment), runs two FlashInfer wrappers, scatters their
outputs into a padded grid and merges it; here ``forward`` is two launches of
``libviewattn.so``:

* ``va_store_kv_rope`` rotates the new keys to their block-relative position
  and scatters K and V into the pool (reference ``attention.py:645-649``);
* ``va_attention`` walks the planned work items: page-table gather, query
  re-rotation per segment inside the kernel, online softmax, and the LSE merge
  across KV chunks and segments (reference ``attention.py:652-752``).

Semantics kept from the reference: keys are stored at block-relative RoPE
positions and never re-rotated; the query of row ``w`` is rotated by
``total_span - prefix_span - 1`` for each segment; segment lengths count this
step's appended tokens, which are stored before any attention runs; a writer
whose block is outside its view still sees its own new token.
"""

from __future__ import annotations

import os
from dataclasses import dataclass, field
from typing import Dict, List, Literal, Optional, Sequence

import numpy as np
import torch

from .. import native
from .attention_metadata import page_numbers_array, upload_page_indices
from .rope_correction import rope_rows


class BaseAttnMetadata:
    """Interface of the reference ``BaseAttnMetadata`` (``attention/base.py:12-15``)."""

    def get_last_indices(self, bs: int) -> torch.Tensor:  # pragma: no cover - interface
        raise NotImplementedError


@dataclass
class LaunchPlan:
    """Device copy of one launch's tables plus the host header ``va_attention``
    needs; everything referenced here must outlive the launch."""

    header: np.ndarray  # int32 [PLAN_HEADER_WORDS], host
    blob: torch.Tensor  # int32 device: work items, links, merge lists
    kv_indices: torch.Tensor  # int32 device
    counts: native.VaPlanCounts
    workspace: Optional[torch.Tensor]


@dataclass
class SharedCacheAttnMetadata(BaseAttnMetadata):
    # attention layers divert to ``shared_cache_op.forward`` when they find this attribute
    shared_cache_op: "SharedCacheAttention"
    sub_worker: torch.Tensor  # int64 [N_sub]: query/output row of each (row, segment) sub-row
    sub_loc: torch.Tensor  # int64 [N_sub] or [3, N_sub]: rotation position of each sub-row
    pad_slot: torch.Tensor  # int64 [N_sub]: row * max_segments + segment
    num_workers: int  # output rows
    max_segments: int
    n_main: int = 0  # decode: paged sub-requests
    n_aux: int = 0  # decode: single-slot sub-requests (writer outside its own view)
    n_ctx_rows: int = 0  # prefill: sub-rows of the non-causal context part
    last_indices: Optional[torch.Tensor] = None
    phase: Literal["decode", "prefill_batch", "mixed"] = "decode"
    _plan_refs: tuple = field(default=(), repr=False)
    graph_buffers: object | None = field(default=None, repr=False)
    # host copies of the planned tables, keyed like the reference's FlashInfer plan() kwargs
    main_plan: Optional[dict] = field(default=None, repr=False)
    aux_plan: Optional[dict] = field(default=None, repr=False)
    launch: Optional[LaunchPlan] = field(default=None, repr=False)

    def get_last_indices(self, bs: int) -> torch.Tensor:
        if self.phase in ("prefill_batch", "mixed"):
            assert self.last_indices is not None
            return self.last_indices
        return torch.arange(bs, device=self.sub_worker.device)


@dataclass
class PrefillSpec:
    """One request of a batched view-conditioned prefill (reference
    ``attention.py:98-115``): the non-empty blocks it reads in view order, the
    write block's complete post-write page list, the number of new tokens, how
    many tokens / how much mRoPE span the write block already held, and the new
    tokens' zero-based 3-D positions when they contain an image."""

    context: list
    self_page_starts: torch.Tensor
    num_new: int
    self_prefix_len: int = 0
    self_prefix_span: Optional[int] = None
    mrope_rel: Optional[torch.Tensor] = None


def _rel_positions(mrope_rel: Optional[torch.Tensor], num_new: int, use_3d: bool) -> torch.Tensor:
    """Zero-based positions of the new tokens: ``[S]``, or ``[3, S]`` as soon as
    any request of the batch is 3-D (reference ``attention.py:118-127``)."""
    if mrope_rel is None:
        base = torch.arange(num_new, dtype=torch.int64)
        return base.unsqueeze(0).expand(3, -1) if use_3d else base
    rel = mrope_rel.to(device="cpu", dtype=torch.int64)
    assert rel.shape == (3, num_new), f"mrope_rel must be [3, {num_new}], got {tuple(rel.shape)}"
    return rel


def _i32(values) -> torch.Tensor:
    return torch.tensor(values, dtype=torch.int32, device="cpu")


def _cumulative(counts: Sequence[int]) -> torch.Tensor:
    out = torch.zeros(len(counts) + 1, dtype=torch.int32)
    if counts:
        out[1:] = torch.tensor(counts, dtype=torch.int64).cumsum(0).to(torch.int32)
    return out


_KERNELS = {"auto": native.VA_KERNEL_AUTO, "generic": native.VA_KERNEL_GENERIC, "mfma": native.VA_KERNEL_MFMA}


class SharedCacheAttention:
    """View attention over a paged KV pool.  ``kv_cache`` needs ``k_cache(layer)``
    and ``v_cache(layer)`` returning ``[num_pages, page_size, kv_heads, head_dim]``
    tensors on ``device``; ``cos_sin_cache`` is the fp32 ``[max_pos, rotary_dim]``
    cos|sin table (unused when ``mrope_section`` is set)."""

    def __init__(
        self,
        kv_cache,
        cos_sin_cache: torch.Tensor,
        num_qo_heads: int,
        num_kv_heads: int,
        head_dim: int,
        page_size: int,
        dtype: torch.dtype,
        device: torch.device,
        rotary_dim: int | None = None,
        mrope_section: tuple | None = None,
        rope_base: float | None = None,
        kernel: str | None = None,
        fused_store: bool = True,
    ) -> None:
        self.kv_cache = kv_cache
        # False: new rows reach the pool through ``kv_cache.store_kv`` as in the reference
        # (``attention.py:645-649``: rotate, then store), one launch more per step -- for a pool whose
        # ``store_kv`` does more than copy rows (hooks, a storage format of its own behind it)
        self.fused_store = fused_store
        self.num_qo_heads = num_qo_heads
        self.num_kv_heads = num_kv_heads
        self.head_dim = head_dim
        self.rotary_dim = head_dim if rotary_dim is None else rotary_dim
        self.mrope_section = mrope_section
        self.page_size = page_size
        self.dtype = dtype
        self.device = torch.device(device)
        self.cos_sin_cache = cos_sin_cache
        self._mrope_inv_freq = None
        if mrope_section is not None:
            assert rope_base is not None, "mrope_section needs rope_base"
            exponent = torch.arange(0, self.rotary_dim, 2, dtype=torch.float32, device=self.device) / self.rotary_dim
            self._mrope_inv_freq = (1.0 / (rope_base ** exponent)).contiguous()
        kernel = kernel or os.environ.get("VIEWATTN_KERNEL", "auto")
        if kernel not in _KERNELS:
            raise ValueError(f"kernel must be one of {sorted(_KERNELS)}, got {kernel!r}")
        if kernel == "auto" and self.rotary_dim % 16:
            kernel = "generic"  # the matrix-core kernel rotates queries in 8-element pieces
        self.kernel = kernel
        # planner knobs (0 = let the planner choose); VIEWATTN_PLAN="kv_chunk=1024,target_items=768" overrides
        knobs = dict(q_tile=0, kv_chunk=0, target_items=0, wide_tile=0)
        for part in filter(None, os.environ.get("VIEWATTN_PLAN", "").split(",")):
            name, _, value = part.partition("=")
            if name.strip() not in knobs:
                raise ValueError(f"VIEWATTN_PLAN: unknown knob {name!r} (known: {sorted(knobs)})")
            knobs[name.strip()] = int(value)
        self.plan_params = native.VaPlanParams(_KERNELS[kernel], knobs["q_tile"], knobs["kv_chunk"],
                                               knobs["target_items"], knobs["wide_tile"])
        self._shape = native.make_shape(num_qo_heads, num_kv_heads, head_dim, page_size, dtype)
        self._rope_desc: Optional[native.VaRope] = None
        self._workspace: Optional[torch.Tensor] = None
        self._workspace_prepared = False
        self._plan_scratch = np.empty(1 << 16, dtype=np.int32)  # host scratch of the planner, grown on demand
        self._checked_layers = set()
        if fused_store:
            self._check_pool_layout()

    def _check_pool_layout(self, layer_id: int = 0) -> None:
        """``forward`` writes new K/V rows into ``k_cache(layer)`` / ``v_cache(layer)`` itself (the key
        rotation is fused into the store) instead of calling ``kv_cache.store_kv`` as the reference
        does (``attention.py:649``).  That is only the same thing for a pool that is a plain
        ``[num_pages, page_size, kv_heads, head_dim]`` array of the op's dtype, so a pool of any other
        layout is refused -- when the op is built, and again for every layer it stores into -- rather
        than silently written wrongly.  A planner-only stand-in without layers (the reference's
        planner tests pass a bare namespace) has nothing to check."""
        want = (self.page_size, self.num_kv_heads, self.head_dim)
        for name in ("k_cache", "v_cache"):
            getter = getattr(self.kv_cache, name, None)
            layer = getter(layer_id) if callable(getter) else None
            if layer is None:
                continue
            if layer.dim() != 4 or tuple(layer.shape[1:]) != want:
                raise ValueError(f"kv_cache.{name}({layer_id}) must be [num_pages, {want[0]}, {want[1]}, {want[2]}], "
                                 f"got {tuple(layer.shape)}")
            if layer.dtype != self.dtype or not layer.is_contiguous():
                raise ValueError(f"kv_cache.{name}({layer_id}) must be a contiguous {self.dtype} tensor, got "
                                 f"{layer.dtype}, contiguous={layer.is_contiguous()}")

    # ------------------------------------------------------------------
    # rotation
    # ------------------------------------------------------------------
    def _rope_descriptor(self) -> native.VaRope:
        if self._rope_desc is None and self.rotary_dim == 0:
            # nothing rotates (queries and keys arrive rotated): no table is needed
            self._rope_desc = native.VaRope(native.VA_ROPE_TABLE, 0, None, 0, 0, 0, None)
        if self._rope_desc is None:
            table = None
            if self.mrope_section is None:
                table = self.cos_sin_cache
                if table.device != self.device or table.dtype != torch.float32 or not table.is_contiguous():
                    table = table.to(device=self.device, dtype=torch.float32).contiguous()
                self._table = table  # keep the converted copy alive
            self._rope_desc = native.make_rope(self.rotary_dim, table, self._mrope_inv_freq, self.mrope_section)
        return self._rope_desc

    def _rope(self, x: torch.Tensor, corrections: torch.Tensor) -> torch.Tensor:
        """Block-relative rotation of ``x [N, heads, head_dim]`` (reference
        ``_rope`` / ``_rope_mrope``, ``attention.py:241-280``); partial rotary
        passes the tail dims through."""
        return rope_rows(x, corrections, self._rope_descriptor())

    # ------------------------------------------------------------------
    # workspace
    # ------------------------------------------------------------------
    def _ensure_workspace(self, nbytes: int) -> Optional[torch.Tensor]:
        if nbytes == 0:
            return self._workspace
        if self._workspace is None or self._workspace.numel() < nbytes:
            if self._workspace_prepared:
                raise RuntimeError("Attention workspace was fixed by prepare_workspace and is too small")
            self._workspace = torch.empty(max(nbytes, 1 << 20), dtype=torch.uint8, device=self.device)
        return self._workspace

    def prepare_workspace(self, profiles) -> None:
        """Reserve the scratch of the whole catalogue of fixed-capacity profiles once, before any
        capture (reference ``attention.py:212-239``).  A profile's ``workspace_requirements()``
        lists ``(consumer, float_bytes, int_bytes)`` entries: every consumer shares one arena of
        the largest ``float_bytes`` (here: the partial softmax states of a launch) and owns
        ``int_bytes`` of table storage of its own, both handed over through
        ``consumer.reset_workspace_buffer(arena, ints)``.  Everything is allocated before the
        first consumer is rebound, so an allocation that fails leaves the op and every consumer
        as they were, not prepared."""
        profiles = tuple(profiles)
        if not profiles:
            return
        if self._workspace_prepared or (self.device.type == "cuda" and torch.cuda.is_current_stream_capturing()):
            raise RuntimeError("Attention workspace must be prepared once before capture")
        if any(p.attention is not self for p in profiles):
            raise ValueError("Attention workspace profiles must belong to this instance")
        wanted = [entry for p in profiles for entry in p.workspace_requirements()]
        arena = self._workspace
        size = max([0 if arena is None else arena.numel()] + [int(float_bytes) for _, float_bytes, _ in wanted])
        if arena is None or size > arena.numel():
            arena = torch.empty(size, dtype=torch.uint8, device=self.device)
        tables = [torch.empty(max(16, int(int_bytes)), dtype=torch.uint8, device=self.device)
                  for _, _, int_bytes in wanted]
        for (consumer, _, _), ints in zip(wanted, tables):
            consumer.reset_workspace_buffer(arena, ints)
        self._workspace = arena
        self._workspace_prepared = True

    # ------------------------------------------------------------------
    # planning
    # ------------------------------------------------------------------
    def _build_launch(self, qo_indptr, kv_indptr, kv_indices_host, seq_lens, flags, chain, sub_worker_host,
                      n_rows: int, kv_indices_dev: torch.Tensor, refs: list) -> LaunchPlan:
        """Run the native work decomposition over the planned tables and upload
        the resulting plan blob."""
        arrays = [np.ascontiguousarray(a, dtype=np.int32) for a in (qo_indptr, kv_indptr, kv_indices_host,
                                                                    seq_lens, flags, chain)]
        sw = np.ascontiguousarray(sub_worker_host, dtype=np.int64)
        n_sub = len(arrays[3])
        subs = native.VaSubRequests(
            n_sub, len(sw), n_rows,
            arrays[0].ctypes.data, arrays[1].ctypes.data, arrays[2].ctypes.data if arrays[2].size else None,
            arrays[3].ctypes.data, arrays[4].ctypes.data, arrays[5].ctypes.data,
            sw.ctypes.data if sw.size else None)
        # one pass of the planner: build into a scratch that is normally large enough, then copy
        # the blob to pinned staging of its exact size
        counts = native.VaPlanCounts()
        scratch = self._plan_scratch
        rc = native.lib.va_plan_build(subs, self._shape, self.plan_params, scratch.ctypes.data, scratch.size, counts)
        if rc == native.VA_ERR_CAPACITY and counts.plan_words > scratch.size:
            scratch = self._plan_scratch = np.empty(2 * counts.plan_words, dtype=np.int32)
            rc = native.lib.va_plan_build(subs, self._shape, self.plan_params, scratch.ctypes.data, scratch.size,
                                          counts)
        native.check(rc)
        pin = self.device.type == "cuda"
        host = torch.empty(counts.plan_words, dtype=torch.int32, pin_memory=pin)
        host.numpy()[:] = scratch[: counts.plan_words]
        blob = host.to(self.device, non_blocking=True)
        refs.extend((host, blob))
        header = host[: native.PLAN_HEADER_WORDS].numpy().copy()
        return LaunchPlan(header, blob, kv_indices_dev, counts, self._ensure_workspace(counts.workspace_bytes))

    def _walk_decode(self, group, new_page_for_block, new_token_slots):
        """Sub-requests of one decode step: per worker one paged sub-request per
        non-empty view block, plus a single-slot one when it writes outside its
        view (reference ``attention.py:326-370``).  The (worker, block) pairs are
        walked once to number the distinct blocks; lengths, spans, rotation
        offsets and segment slots are then array arithmetic over those numbers.
        Returns ``main`` / ``aux`` tables (int64 arrays, ``pages`` a list of int32
        arrays) in the reference's order, and the largest segment count."""
        W = group.num_workers
        assert W > 0
        P = self.page_size
        views, targets = group.cache_structure, group.write_to

        number: Dict[int, int] = {}  # id(block) -> index into `blocks`
        blocks: list = []
        flat: List[int] = []  # block number of every (worker, view position), worker-major
        counts = np.empty(W, dtype=np.int64)
        for w, view in enumerate(views):
            counts[w] = len(view)
            for b in view:
                k = number.get(id(b))
                if k is None:
                    k = number[id(b)] = len(blocks)
                    blocks.append(b)
                flat.append(k)
        n_blocks = len(blocks)
        tokens = np.fromiter((b.num_tokens for b in blocks), dtype=np.int64, count=n_blocks)
        spans = np.fromiter((b.mrope_span for b in blocks), dtype=np.int64, count=n_blocks)
        grow = np.fromiter((id(b) in new_page_for_block for b in blocks), dtype=np.int64, count=n_blocks)
        tokens += grow  # this step's appends are stored before any attention runs
        spans += grow

        flat_arr = np.asarray(flat, dtype=np.int64)
        worker = np.repeat(np.arange(W, dtype=np.int64), counts)
        first = np.concatenate(([0], np.cumsum(counts)[:-1]))  # first pair of each worker
        span = spans[flat_arr]
        length = tokens[flat_arr]
        ahead = np.cumsum(span) - span  # span of all pairs before this one ...
        total = np.bincount(worker, weights=span, minlength=W).astype(np.int64)  # exact: spans are far below 2^53
        base = np.zeros(W, dtype=np.int64)
        has_view = counts > 0
        base[has_view] = ahead[first[has_view]]
        ahead -= base[worker]  # ... and of the blocks ahead of it in its own view
        live = length > 0
        seen = np.cumsum(live) - live
        seg_base = np.zeros(W, dtype=np.int64)
        seg_base[has_view] = seen[first[has_view]]
        segments = np.bincount(worker[live], minlength=W)

        snapshot: Dict[int, np.ndarray] = {}
        page_of_block: List[Optional[np.ndarray]] = [None] * n_blocks
        pages = []
        for k in flat_arr[live].tolist():
            got = page_of_block[k]
            if got is None:
                b = blocks[k]
                got = page_of_block[k] = page_numbers_array(b, snapshot, new_page_for_block.get(id(b)))
            pages.append(got)
        n_pages = np.fromiter((len(p) for p in pages), dtype=np.int64, count=len(pages))
        main = {"worker": worker[live], "loc": (total[worker] - ahead - 1)[live], "slot": (seen - seg_base[worker])[live],
                "pages": pages, "n_pages": n_pages, "len": length[live]}
        main["last"] = main["len"] - (n_pages - 1) * P

        # a writer whose block is outside its view still attends to the token it writes, at distance 0
        target_no = np.fromiter((number.get(id(t), -1) for t in targets), dtype=np.int64, count=W)
        inside = np.zeros(W, dtype=bool)
        inside[worker[flat_arr == target_no[worker]]] = True
        outside = np.nonzero(~inside)[0]
        aux = {"worker": outside, "loc": np.fromiter((targets[w].mrope_span for w in outside.tolist()), dtype=np.int64,
                                                      count=len(outside)),
               "slot": segments[outside], "kv": np.zeros(0, dtype=np.int64)}
        if len(outside):
            aux["kv"] = new_token_slots.cpu().numpy().astype(np.int64)[outside]
            segments = segments.copy()
            segments[outside] += 1
        return main, aux, int(segments.max())

    def prepare(
        self,
        group,
        new_page_for_block: Dict[int, Optional[int]],
        new_token_slots: torch.Tensor,
        graph_buffers=None,
    ) -> SharedCacheAttnMetadata:
        """Plan one decode step (reference ``attention.py:282-448``).

        ``new_page_for_block`` maps ``id(write_block)`` to the page-start slot of
        the page this step's token opens (``None`` if it fits the last page); its
        keys are the blocks written this step.  ``new_token_slots [W]`` are the
        slots of the new tokens.  Blocks are not modified.
        """
        W = group.num_workers
        P = self.page_size
        main, aux, max_segments = self._walk_decode(group, new_page_for_block, new_token_slots)

        if graph_buffers is not None:
            return graph_buffers.plan(main["worker"], main["loc"], main["slot"], main["pages"], main["n_pages"],
                                      main["len"], main["last"], aux["worker"], aux["loc"], aux["kv"])

        n_main, n_aux = len(main["worker"]), len(aux["worker"])
        refs: List[torch.Tensor] = []
        parts = list(main["pages"])
        if n_aux:
            parts.append(aux["kv"])
        kv_indices = upload_page_indices(parts, self.device, refs)
        kv_host = refs[0]
        n_main_entries = int(main["n_pages"].sum())
        main_indptr = np.concatenate(([0], np.cumsum(main["n_pages"])))

        main_plan = aux_plan = None
        if n_main:
            main_plan = dict(indptr=torch.from_numpy(main_indptr.astype(np.int32)), indices=kv_host[:n_main_entries],
                             last_page_len=torch.from_numpy(main["last"].astype(np.int32)),
                             seq_lens=torch.from_numpy(main["len"].astype(np.int32)), page_size=P)
        if n_aux:
            aux_plan = dict(indptr=torch.arange(n_aux + 1, dtype=torch.int32), indices=kv_host[n_main_entries:],
                            last_page_len=torch.ones(n_aux, dtype=torch.int32),
                            seq_lens=torch.ones(n_aux, dtype=torch.int32), page_size=1)

        sub_worker = np.concatenate([main["worker"], aux["worker"]])
        sub_loc = np.concatenate([main["loc"], aux["loc"]])
        pad_slot = sub_worker * max_segments + np.concatenate([main["slot"], aux["slot"]])
        n_sub = n_main + n_aux

        launch = self._build_launch(
            qo_indptr=np.arange(n_sub + 1),
            kv_indptr=np.concatenate([main_indptr, n_main_entries + 1 + np.arange(n_aux)]),
            kv_indices_host=kv_host.numpy(),
            seq_lens=np.concatenate([main["len"], np.ones(n_aux, dtype=np.int64)]),
            flags=np.concatenate([np.zeros(n_main, dtype=np.int32), np.full(n_aux, native.VA_SUB_SLOTS, dtype=np.int32)]),
            chain=np.full(n_sub, -1, dtype=np.int32),
            sub_worker_host=sub_worker,
            n_rows=W, kv_indices_dev=kv_indices, refs=refs)

        dev_sub_worker, dev_sub_loc, dev_pad = self._upload_i64([sub_worker, sub_loc, pad_slot], refs)
        meta = SharedCacheAttnMetadata(
            shared_cache_op=self, sub_worker=dev_sub_worker, sub_loc=dev_sub_loc, pad_slot=dev_pad,
            num_workers=W, max_segments=max_segments, n_main=n_main, n_aux=n_aux,
            main_plan=main_plan, aux_plan=aux_plan, launch=launch)
        meta._plan_refs = tuple(refs)
        return meta

    def _upload_i64(self, rows: Sequence, refs: list) -> List[torch.Tensor]:
        """One pinned staging tensor and one async copy for several equally long
        int64 tables; returns the device rows."""
        host = torch.from_numpy(np.stack([np.asarray(r, dtype=np.int64) for r in rows]))
        if self.device.type == "cuda":
            host = host.pin_memory()
        dev = host.to(self.device, non_blocking=True)
        refs.extend((host, dev))
        return [dev[i] for i in range(len(rows))]

    def _walk_prefill(self, specs, use_3d: bool):
        """Sub-requests of a batched prefill: per request one non-causal sub-request
        per context block and one causal sub-request over its own block."""
        P = self.page_size
        max_segments = max(len(s.context) + 1 for s in specs)
        snapshot: Dict[int, np.ndarray] = {}

        ctx = {"rows": [], "slot": [], "loc": [], "pages": [], "n_pages": [], "q": [], "len": [], "last": [],
               "chain": []}
        own = {"rows": [], "slot": [], "loc": [], "pages": [], "n_pages": [], "q": [], "len": [], "last": [],
               "chain": []}
        last_indices: List[int] = []
        offset = 0
        for r, spec in enumerate(specs):
            S = int(spec.num_new)
            assert S > 0
            T = int(spec.self_prefix_len)
            T_span = T if spec.self_prefix_span is None else int(spec.self_prefix_span)
            spans = [b.mrope_span for b in spec.context]
            first_new = sum(spans) + T_span  # running position of the first new token
            rows = np.arange(offset, offset + S, dtype=np.int64)
            rel = _rel_positions(spec.mrope_rel, S, use_3d)
            ahead = 0
            for j, (block, span) in enumerate(zip(spec.context, spans)):
                assert block.num_tokens > 0, "context blocks must be non-empty"
                ctx["rows"].append(rows)
                ctx["slot"].append(np.full(S, j, dtype=np.int64))
                ctx["loc"].append(rel + (first_new - ahead))
                ctx["pages"].append(page_numbers_array(block, snapshot))
                ctx["n_pages"].append(block.num_pages)
                ctx["q"].append(S)
                ctx["len"].append(block.num_tokens)
                ctx["last"].append(block.last_page_len)
                ctx["chain"].append(r)
                ahead += span
            pages = [start // P for start in spec.self_page_starts.cpu().tolist()]
            own["rows"].append(rows)
            own["slot"].append(np.full(S, len(spec.context), dtype=np.int64))
            own["loc"].append(rel + T_span)
            own["pages"].append(pages)
            own["n_pages"].append(len(pages))
            own["q"].append(S)
            own["len"].append(T + S)
            own["last"].append(T + S - (len(pages) - 1) * P)
            own["chain"].append(r)
            last_indices.append(offset + S - 1)
            offset += S

        return ctx, own, last_indices, offset, max_segments

    def prepare_prefill_batch(self, specs: List[PrefillSpec], graph_buffers=None) -> SharedCacheAttnMetadata:
        """Plan several view-conditioned prefills as one launch, request-major
        (reference ``attention.py:450-622``).  Request ``r`` owns output rows
        ``[offset_r, offset_r + num_new_r)``; its new tokens attend fully to each
        context block (sized before this step's writes) and causally to their
        own block, prefix included."""
        assert specs, "prepare_prefill_batch needs at least one request"
        if graph_buffers is not None:
            return graph_buffers.plan(specs)
        P = self.page_size
        use_3d = any(s.mrope_rel is not None for s in specs)
        ctx, own, last_indices, offset, max_segments = self._walk_prefill(specs, use_3d)

        n_rows = offset
        sub_gather = np.concatenate(ctx["rows"] + own["rows"])
        sub_slot = np.concatenate(ctx["slot"] + own["slot"])
        sub_loc = torch.cat(ctx["loc"] + own["loc"], dim=1 if use_3d else 0)
        pad_slot = sub_gather * max_segments + sub_slot
        n_ctx_rows = int(sum(ctx["q"]))

        refs: List[torch.Tensor] = []
        kv_indices = upload_page_indices(ctx["pages"] + own["pages"], self.device, refs)
        kv_host = refs[0]
        n_ctx_entries = sum(ctx["n_pages"])
        ctx_plan = None
        if ctx["q"]:
            ctx_plan = dict(qo_indptr=_cumulative(ctx["q"]), paged_kv_indptr=_cumulative(ctx["n_pages"]),
                            paged_kv_indices=kv_host[:n_ctx_entries], paged_kv_last_page_len=_i32(ctx["last"]),
                            seq_lens=_i32(ctx["len"]), max_token_per_sequence=max(ctx["q"]), causal=False,
                            page_size=P)
        self_plan = dict(qo_indptr=_cumulative(own["q"]), paged_kv_indptr=_cumulative(own["n_pages"]),
                         paged_kv_indices=kv_host[n_ctx_entries:], paged_kv_last_page_len=_i32(own["last"]),
                         seq_lens=_i32(own["len"]), max_token_per_sequence=max(own["q"]), causal=True,
                         page_size=P)

        n_ctx, n_self = len(ctx["q"]), len(own["q"])
        launch = self._build_launch(
            qo_indptr=np.cumsum([0] + ctx["q"] + own["q"]),
            kv_indptr=np.cumsum([0] + ctx["n_pages"] + own["n_pages"]),
            kv_indices_host=kv_host.numpy(),
            seq_lens=ctx["len"] + own["len"],
            flags=[0] * n_ctx + [native.VA_SUB_CAUSAL] * n_self,
            chain=ctx["chain"] + own["chain"],
            sub_worker_host=sub_gather,
            n_rows=n_rows, kv_indices_dev=kv_indices, refs=refs)

        def to_dev(t: torch.Tensor) -> torch.Tensor:
            host = t.contiguous()
            if self.device.type == "cuda":
                host = host.pin_memory()
            dev = host.to(self.device, non_blocking=True)
            refs.extend((host, dev))
            return dev

        meta = SharedCacheAttnMetadata(
            shared_cache_op=self,
            sub_worker=to_dev(torch.from_numpy(sub_gather)),
            sub_loc=to_dev(sub_loc),
            pad_slot=to_dev(torch.from_numpy(pad_slot)),
            num_workers=n_rows, max_segments=max_segments, n_ctx_rows=n_ctx_rows,
            last_indices=to_dev(torch.tensor(last_indices, dtype=torch.int64)),
            phase="prefill_batch", main_plan=ctx_plan, aux_plan=self_plan, launch=launch)
        meta._plan_refs = tuple(refs)
        return meta

    def prepare_mixed(self, group, new_page_for_block: Dict[int, Optional[int]], new_token_slots: torch.Tensor,
                      specs: List[PrefillSpec]) -> SharedCacheAttnMetadata:
        """Plan one decode step AND a batch of view-conditioned prefill chunks as a
        single launch (a continuous batch).  Output rows are the ``W`` decode
        workers followed by the prefill tokens, request-major; ``forward`` takes
        q/k/v, ``positions`` and ``out_loc`` in that row order.  The two parts
        keep their own semantics (``prepare`` / ``prepare_prefill_batch``): all new
        K/V rows are stored before any attention runs, decode lengths count this
        step's decode appends, prefill context lengths are pre-write.  The
        reference runs the two as separate forwards (``session.decode_step`` /
        ``prefill_batch``); nothing in its tables changes, they are concatenated.
        """
        assert specs, "prepare_mixed needs at least one prefill request (use prepare otherwise)"
        W = group.num_workers
        assert W > 0
        P = self.page_size
        use_3d = any(s.mrope_rel is not None for s in specs)
        main, aux, seg_d = self._walk_decode(group, new_page_for_block, new_token_slots)
        ctx, own, last_indices, n_new, seg_p = self._walk_prefill(specs, use_3d)
        M = max(seg_d, seg_p)
        n_main, n_aux, n_ctx, n_self = len(main["worker"]), len(aux["worker"]), len(ctx["q"]), len(own["q"])

        refs: List[torch.Tensor] = []
        parts = list(main["pages"]) + ([aux["kv"]] if n_aux else []) + ctx["pages"] + own["pages"]
        kv_indices = upload_page_indices(parts, self.device, refs)
        kv_host = refs[0]
        kv_counts = main["n_pages"].tolist() + [1] * n_aux + ctx["n_pages"] + own["n_pages"]

        dec_worker = np.concatenate([main["worker"], aux["worker"]])
        dec_slot = np.concatenate([main["slot"], aux["slot"]])
        dec_loc = torch.from_numpy(np.concatenate([main["loc"], aux["loc"]]))
        pre_rows = np.concatenate(ctx["rows"] + own["rows"]) + W
        pre_slot = np.concatenate(ctx["slot"] + own["slot"])
        pre_loc = torch.cat(ctx["loc"] + own["loc"], dim=1 if use_3d else 0)
        if use_3d:
            dec_loc = dec_loc.unsqueeze(0).expand(3, -1)
        sub_worker = np.concatenate([dec_worker, pre_rows])
        sub_loc = torch.cat([dec_loc, pre_loc], dim=1 if use_3d else 0)
        pad_slot = sub_worker * M + np.concatenate([dec_slot, pre_slot])

        launch = self._build_launch(
            qo_indptr=np.cumsum([0] + [1] * (n_main + n_aux) + ctx["q"] + own["q"]),
            kv_indptr=np.cumsum([0] + kv_counts),
            kv_indices_host=kv_host.numpy(),
            seq_lens=main["len"].tolist() + [1] * n_aux + ctx["len"] + own["len"],
            flags=[0] * n_main + [native.VA_SUB_SLOTS] * n_aux + [0] * n_ctx + [native.VA_SUB_CAUSAL] * n_self,
            chain=[-1] * (n_main + n_aux) + ctx["chain"] + own["chain"],
            sub_worker_host=sub_worker,
            n_rows=W + n_new, kv_indices_dev=kv_indices, refs=refs)

        def to_dev(t: torch.Tensor) -> torch.Tensor:
            host = t.contiguous()
            if self.device.type == "cuda":
                host = host.pin_memory()
            dev = host.to(self.device, non_blocking=True)
            refs.extend((host, dev))
            return dev

        last = torch.cat([torch.arange(W, dtype=torch.int64), torch.tensor(last_indices, dtype=torch.int64) + W])
        meta = SharedCacheAttnMetadata(
            shared_cache_op=self, sub_worker=to_dev(torch.from_numpy(sub_worker)), sub_loc=to_dev(sub_loc),
            pad_slot=to_dev(torch.from_numpy(pad_slot)), num_workers=W + n_new, max_segments=M,
            n_main=n_main, n_aux=n_aux, n_ctx_rows=int(sum(ctx["q"])), last_indices=to_dev(last),
            phase="mixed", launch=launch)
        meta._plan_refs = tuple(refs)
        return meta

    # ------------------------------------------------------------------
    # execution
    # ------------------------------------------------------------------
    def store_new_kv(self, k: torch.Tensor, v: torch.Tensor, layer_id: int, batch) -> None:
        """Rotate the new keys to their block-relative positions and write K and
        V rows to ``batch.out_loc`` (negative slots are skipped)."""
        native.require_device(k, "k")
        W = k.shape[0]
        if W == 0:
            return
        Hkv, D = self.num_kv_heads, self.head_dim
        key_pos = batch.positions if batch.mrope_positions is None else batch.mrope_positions
        key_pos = key_pos.to(device=self.device, dtype=torch.int64)
        if not self.fused_store:
            k_rot = self._rope(k.reshape(W, Hkv, D), key_pos)
            self.kv_cache.store_kv(k_rot.view(W, Hkv * D), v.reshape(W, Hkv * D), batch.out_loc, layer_id)
            return
        axis_stride = 0
        if key_pos.dim() == 2:
            key_pos = key_pos.contiguous()
            axis_stride = key_pos.shape[1]
        else:
            key_pos = key_pos.contiguous()
        assert key_pos.shape[-1] == W
        k2 = k.reshape(W, Hkv * D)
        v2 = v.reshape(W, Hkv * D)
        if k2.stride(-1) != 1:
            k2 = k2.contiguous()
        if v2.stride(-1) != 1:
            v2 = v2.contiguous()
        k_pool = self.kv_cache.k_cache(layer_id)
        v_pool = self.kv_cache.v_cache(layer_id)
        if layer_id not in self._checked_layers:
            self._check_pool_layout(layer_id)
            self._checked_layers.add(layer_id)
        out_loc = batch.out_loc
        assert out_loc.dtype in (torch.int32, torch.int64) and out_loc.numel() == W
        out_loc = out_loc.contiguous()
        native.check(native.lib.va_store_kv_rope(
            k2.data_ptr(), v2.data_ptr(), k2.stride(0), v2.stride(0), k_pool.data_ptr(), v_pool.data_ptr(),
            Hkv * D, out_loc.data_ptr(), int(out_loc.dtype == torch.int64), key_pos.data_ptr(), axis_stride,
            W, self._shape, self._rope_descriptor(), native.current_stream_ptr(self.device)))

    def attend(self, q: torch.Tensor, layer_id: int, meta: SharedCacheAttnMetadata,
               return_lse: bool = False, lse_base2: bool = False, out: Optional[torch.Tensor] = None,
               lse: Optional[torch.Tensor] = None, static_scratch: bool = False):
        """Run the planned attention over the pool as it is now; returns
        ``out [rows, Hq*D]`` (and ``lse [rows, Hq]`` fp32 on request).  With
        ``static_scratch`` (and ``out`` / ``lse`` given) the call goes through
        ``va_attention_static`` and allocates nothing: the partial states live in
        the library's own per-GPU array, which bounds the plan's size."""
        native.require_device(q, "q")
        launch = meta.launch
        assert launch is not None, "metadata carries no launch plan"
        W, Hq, D = meta.num_workers, self.num_qo_heads, self.head_dim
        q2 = q.reshape(q.shape[0], Hq * D)
        if q2.stride(-1) != 1:
            q2 = q2.contiguous()
        assert q2.shape[0] >= W and q2.dtype == self.dtype
        if out is None:
            out = torch.empty((W, Hq * D), dtype=self.dtype, device=self.device)
        if lse is None and return_lse:
            lse = torch.empty((W, Hq), dtype=torch.float32, device=self.device)
        assert out.shape == (W, Hq * D) and out.dtype == self.dtype and out.is_contiguous()
        assert lse is None or (lse.shape == (W, Hq) and lse.dtype == torch.float32 and lse.is_contiguous())
        k_pool = self.kv_cache.k_cache(layer_id)
        v_pool = self.kv_cache.v_cache(layer_id)
        sub_loc = meta.sub_loc
        axis_stride = sub_loc.stride(0) if sub_loc.dim() == 2 else 0
        head = (q2.data_ptr(), q2.stride(0), k_pool.data_ptr(), v_pool.data_ptr(), self.num_kv_heads * D,
                launch.blob.data_ptr(), launch.header.ctypes.data, launch.kv_indices.data_ptr(),
                meta.sub_worker.data_ptr(), sub_loc.data_ptr(), axis_stride, out.data_ptr(),
                None if lse is None else lse.data_ptr(), int(lse_base2))
        tail = (self._shape, self._rope_descriptor(), native.current_stream_ptr(self.device))
        if static_scratch:
            native.check(native.lib.va_attention_static(*head, *tail))
        else:
            ws = launch.workspace
            native.check(native.lib.va_attention(*head, None if ws is None else ws.data_ptr(),
                                                 0 if ws is None else ws.numel(), *tail))
        return (out, lse) if return_lse else out

    def forward(self, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, layer_id: int, batch) -> torch.Tensor:
        """``q [W, Hq*D]``, ``k``/``v [W, Hkv*D]`` unrotated; ``batch`` carries
        ``attn_metadata``, ``positions`` (block-relative write positions),
        ``mrope_positions`` (``[3, W]`` or ``None``) and ``out_loc``.  Returns
        ``[W, Hq*D]`` (reference ``attention.py:624-703``)."""
        meta = batch.attn_metadata
        assert isinstance(meta, SharedCacheAttnMetadata)
        self.store_new_kv(k, v, layer_id, batch)
        return self.attend(q, layer_id, meta)

    def forward_with_lse(self, q, k, v, layer_id: int, batch, lse_base2: bool = False):
        """``forward`` that also returns the merged logsumexp ``[W, Hq]``."""
        meta = batch.attn_metadata
        self.store_new_kv(k, v, layer_id, batch)
        return self.attend(q, layer_id, meta, return_lse=True, lse_base2=lse_base2)
