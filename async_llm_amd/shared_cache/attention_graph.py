"""Fixed-capacity plans for view attention that is recorded once and replayed
(HIP graphs).

Drop-in for the reference ``SharedDecodeAttentionBuffers`` /
``SharedPrefillAttentionBuffers`` (``python/minisgl/shared_cache/
attention_graph.py``): same constructors, ``plan`` signatures, capacity errors
and metadata geometry (``sub_worker`` / ``pad_slot`` are fixed, ``sub_loc`` and
``valid`` change per plan).  What a replay must find unchanged differs, though.
The reference pins FlashInfer's table buffers; here the launch geometry is what
``va_attention`` reads from the plan header (workgroups per launch, merge grid,
section offsets), so the buffers hold

* one plan blob of ``va_plan_fixed_words`` words whose header depends on the
  capacity alone (``va_plan_build_fixed`` pads the item lists with empty items),
* one page-index table of ``max_pages`` entries (plus one slot entry per worker
  for decode),
* the sub-row tables of the metadata,

all allocated once; ``plan`` rewrites their contents in place through pinned
staging copies on the current stream.  Unused slots are empty sub-requests
(length 0) rather than dummy pages with masked results: the planner drops them,
and output rows nobody serves come back as zeros.
"""

from __future__ import annotations

from typing import List, Optional

import numpy as np
import torch

from .. import native
from .attention_metadata import page_numbers_array


class _FixedPlanBuffers:
    """Device tables of one fixed-capacity launch and their pinned staging."""

    def __init__(self, attention, limits: native.VaPlanLimits, n_subrows: int, kv_entries: int, use_3d: bool):
        self.attention = attention
        device = attention.device
        self._cuda = device.type == "cuda"
        self.capacity = native.VaPlanCapacity()
        native.check(native.lib.va_plan_capacity(attention._shape, attention.plan_params, limits, self.capacity))
        self.plan_words = int(native.lib.va_plan_fixed_words(self.capacity))
        self.n_subrows = n_subrows
        self.kv_entries = kv_entries

        def pair(shape, dtype):
            host = torch.zeros(shape, dtype=dtype, pin_memory=self._cuda)
            return host, torch.zeros(shape, dtype=dtype, device=device)

        self._blob_host, self.blob = pair(self.plan_words, torch.int32)
        self._kv_host, self.kv_indices = pair(max(kv_entries, 1), torch.int32)
        self._loc_host, self.sub_loc = pair((3, n_subrows) if use_3d else (n_subrows,), torch.int64)
        self._valid_host, self.valid = pair(n_subrows, torch.bool)
        self.event = torch.cuda.Event() if self._cuda else None
        self.counts = native.VaPlanCounts()
        self.header: Optional[np.ndarray] = None
        self.refs: list = []
        self._arena: Optional[torch.Tensor] = None  # the catalogue's shared scratch, once prepare_workspace ran
        self._ints: Optional[torch.Tensor] = None

    def workspace_requirements(self) -> List[tuple]:
        """``[(consumer, float_bytes, int_bytes)]`` as the reference's profiles report them
        (``attention_graph.py:62-72, 176-187``): the scratch of the launch at capacity (the same
        for every plan) and no table storage beyond what the buffers already own."""
        return [(self, int(self.counts.workspace_bytes), 0)]

    def reset_workspace_buffer(self, arena: torch.Tensor, ints: torch.Tensor) -> None:
        """Take the arena ``prepare_workspace`` reserved for the whole catalogue."""
        self._arena, self._ints = arena, ints
        if self.header is not None and getattr(self, "meta", None) is not None and self.meta.launch is not None:
            self.meta.launch = self._launch()

    def _wait_for_staging(self) -> None:
        # the pinned staging tensors are reused: the previous plan's copies must have left them
        if self.event is not None:
            self.event.synchronize()

    def _build(self, qo_indptr, kv_indptr, seq_lens, flags, chain, sub_worker, n_rows: int):
        """Plan the sub-request tables into the staging blob and send blob, page
        indices, positions and the valid mask to their device buffers."""
        tables = [np.ascontiguousarray(a, dtype=np.int32) for a in (qo_indptr, kv_indptr, seq_lens, flags, chain)]
        sw = np.ascontiguousarray(sub_worker, dtype=np.int64)
        subs = native.VaSubRequests(
            len(tables[2]), len(sw), n_rows, tables[0].ctypes.data, tables[1].ctypes.data,
            self._kv_host.data_ptr(), tables[2].ctypes.data, tables[3].ctypes.data, tables[4].ctypes.data,
            sw.ctypes.data)
        rc = native.lib.va_plan_build_fixed(subs, self.attention._shape, self.attention.plan_params, self.capacity,
                                            self._blob_host.data_ptr(), self.plan_words, self.counts)
        if rc == native.VA_ERR_CAPACITY:
            raise ValueError(f"Shared attention exceeds graph plan capacity: {native.lib.va_last_error().decode()}")
        native.check(rc)
        header = self._blob_host[: native.PLAN_HEADER_WORDS].numpy().copy()
        if self.header is None:
            self.header = header
        elif not np.array_equal(header, self.header):
            raise RuntimeError("fixed-capacity plan changed its launch geometry")
        for dev, host in ((self.blob, self._blob_host), (self.kv_indices, self._kv_host),
                          (self.sub_loc, self._loc_host), (self.valid, self._valid_host)):
            dev.copy_(host, non_blocking=True)
        if self.event is not None:
            self.event.record()

    def _launch(self):
        from .attention import LaunchPlan

        need = int(self.counts.workspace_bytes)
        arena = self._arena
        if arena is None or arena.numel() < need:
            arena = self.attention._ensure_workspace(need)
        return LaunchPlan(self.header, self.blob, self.kv_indices, self.counts, arena)


class SharedDecodeAttentionBuffers(_FixedPlanBuffers):
    """Decode metadata for up to ``workers`` rows with ``depth`` view blocks each
    and ``max_pages`` page entries in total (reference ``attention_graph.py:14-121``).

    Sub-row ``worker * depth + slot`` is view block ``slot`` of ``worker``;
    sub-row ``workers * depth + worker`` is the worker's own new token when it
    writes outside its view.  ``dummy_slots`` (one pool slot per worker) fill the
    slot entries of workers without such a token; they are never read.
    """

    def __init__(self, attention, workers: int, depth: int, max_pages: int, dummy_slots: Optional[torch.Tensor] = None):
        from .attention import SharedCacheAttnMetadata

        self.workers, self.depth, self.max_pages = workers, depth, max_pages
        self.main_count = workers * depth
        total = self.main_count + workers
        limits = native.VaPlanLimits(total, total, 0, 0, 0, workers)
        super().__init__(attention, limits, total, max_pages + workers, use_3d=False)
        self.dummy_slots = dummy_slots
        self.dummy_cpu = [0] * workers if dummy_slots is None else dummy_slots.cpu().tolist()
        assert len(self.dummy_cpu) == workers, "one dummy slot per worker"
        device = attention.device
        w = torch.arange(workers, device=device)
        slots = torch.arange(depth, device=device)
        self._sub_worker_host = np.concatenate([np.repeat(np.arange(workers), depth), np.arange(workers)])
        self._qo_indptr = np.arange(total + 1)
        self._flags = np.concatenate([np.zeros(self.main_count, np.int32),
                                      np.full(workers, native.VA_SUB_SLOTS, np.int32)])
        self._chain = np.full(total, -1, np.int32)
        self.meta = SharedCacheAttnMetadata(
            shared_cache_op=attention,
            sub_worker=torch.cat([w.repeat_interleave(depth), w]),
            sub_loc=self.sub_loc,
            pad_slot=torch.cat([(w[:, None] * (depth + 1) + slots).flatten(), w * (depth + 1) + depth]),
            num_workers=workers, max_segments=depth + 1, n_main=self.main_count, n_aux=workers,
            graph_buffers=self)
        # an all-empty plan: the buffers are complete (and capturable) before the first real plan
        self.plan([], [], [], [], [], [], [], [], [], [])

    def plan(self, main_workers, main_locs, main_slots, page_parts, page_counts, seq_lengths, last_pages,
             aux_workers, aux_locs, aux_slots):
        """Fill the buffers for one decode step; arguments as the reference's
        ``plan`` (``attention_graph.py:74-121``).  ``last_pages`` follows from
        the lengths here and is accepted for the interface only."""
        w, d, n_main = self.workers, self.depth, self.main_count
        counts = np.zeros(n_main, dtype=np.int64)
        lengths = np.zeros(n_main + w, dtype=np.int32)
        parts: list = [()] * n_main
        for worker, slot, pages, count, length in zip(main_workers, main_slots, page_parts, page_counts, seq_lengths):
            if slot >= d:
                raise ValueError("Shared attention exceeds graph segment capacity")
            if worker >= w:
                raise ValueError("Shared attention exceeds graph worker capacity")
            i = worker * d + slot
            parts[i], counts[i], lengths[i] = pages, count, length
        n_entries = int(counts.sum())
        if n_entries > self.max_pages:
            raise ValueError("Shared attention exceeds graph page-index capacity")
        if any(worker >= w for worker in aux_workers):
            raise ValueError("Shared attention exceeds graph worker capacity")

        self._wait_for_staging()
        self.refs = []
        kv = self._kv_host.numpy()
        if n_entries:
            np.concatenate([np.asarray(part, dtype=np.int32) for part in parts if len(part)], out=kv[:n_entries])
        kv[n_entries:n_entries + w] = self.dummy_cpu
        loc = self._loc_host.numpy()
        valid = self._valid_host.numpy()
        loc[:] = 0
        valid[:] = False
        if len(main_workers):
            at = np.asarray(main_workers, dtype=np.int64) * d + np.asarray(main_slots, dtype=np.int64)
            loc[at] = main_locs
            valid[at] = True
        for worker, offset, token_slot in zip(aux_workers, aux_locs, aux_slots):
            kv[n_entries + worker] = token_slot
            lengths[n_main + worker] = 1
            loc[n_main + worker] = offset
            valid[n_main + worker] = True
        kv_indptr = np.concatenate([[0], np.cumsum(counts), n_entries + 1 + np.arange(w)])
        self._build(self._qo_indptr, kv_indptr, lengths, self._flags, self._chain, self._sub_worker_host, w)
        self.meta.launch = self._launch()
        return self.meta


class SharedPrefillAttentionBuffers(_FixedPlanBuffers):
    """Batched view-conditioned prefill for up to ``workers`` requests of up to
    ``depth`` context blocks each, ``rows`` new tokens in total and ``max_pages``
    page entries (reference ``attention_graph.py:124-290``).

    Sub-rows ``[0, rows * depth)`` are the (token, context block) pairs in use,
    request-major, then unused ones; sub-rows ``[rows * depth, rows * (depth + 1))``
    are the tokens' causal pass over their own block, so their part of
    ``sub_worker`` never changes.  ``dummy_slots`` is accepted for the interface:
    unused request slots are empty here and read nothing.
    """

    def __init__(self, attention, workers: int, depth: int, rows: int, max_pages: int,
                 dummy_slots: Optional[torch.Tensor] = None):
        from .attention import SharedCacheAttnMetadata

        self.workers, self.depth, self.rows = workers, depth, rows
        self.max_pages, self.ctx_rows = max_pages, rows * depth
        self.use_3d = attention.mrope_section is not None
        total = rows * (depth + 1)
        limits = native.VaPlanLimits(0, 0, workers, depth + 1, rows, rows)
        super().__init__(attention, limits, total, max_pages, use_3d=self.use_3d)
        device = attention.device
        self._cuda_pair = lambda n: (torch.zeros(n, dtype=torch.int64, pin_memory=self._cuda),
                                     torch.zeros(n, dtype=torch.int64, device=device))
        self._sub_worker_host, sub_worker = self._cuda_pair(total)
        self._pad_host, pad_slot = self._cuda_pair(total)
        self._last_host, last_indices = self._cuda_pair(workers)
        self._sub_worker_host[self.ctx_rows:] = torch.arange(rows)
        self._all_slots = np.arange(total)
        self.used_ctx_rows, self.used_self_rows = 0, 0
        self.meta = SharedCacheAttnMetadata(
            shared_cache_op=attention, sub_worker=sub_worker, sub_loc=self.sub_loc, pad_slot=pad_slot,
            num_workers=rows, max_segments=depth + 1, n_ctx_rows=self.ctx_rows, last_indices=last_indices,
            phase="prefill_batch", graph_buffers=self)
        self.plan([])

    def plan(self, specs):
        """Fill the buffers for one batch of ``PrefillSpec`` s (reference
        ``attention_graph.py:196-290``); an empty list plans a launch that only
        clears its output rows."""
        from .attention import _rel_positions

        a, w, d, r = self.attention, self.workers, self.depth, self.rows
        if len(specs) > w or sum(s.num_new for s in specs) > r or any(len(s.context) > d for s in specs):
            raise ValueError("Shared prefill exceeds graph request/row/segment capacity")
        P = a.page_size
        snapshot: dict = {}
        # sub-requests: workers * depth context slots, an empty one that owns the unused context
        # sub-rows, workers self slots, an empty one that owns the unused self sub-rows
        n_sub = w * d + 1 + w + 1
        q_len = np.zeros(n_sub, dtype=np.int64)
        lengths = np.zeros(n_sub, dtype=np.int32)
        flags = np.zeros(n_sub, dtype=np.int32)
        flags[w * d + 1:w * d + 1 + w] = native.VA_SUB_CAUSAL
        chain = np.full(n_sub, -1, dtype=np.int32)
        pages: list = [()] * n_sub
        gather, slots, locations = [], [], []
        self_loc = torch.zeros((3, r) if self.use_3d else (r,), dtype=torch.int64)
        self_slots = np.arange(r, dtype=np.int64) * (d + 1) + d
        last_rows = [0] * w
        offset = 0
        for worker, spec in enumerate(specs):
            n = int(spec.num_new)
            assert n > 0
            source = np.arange(offset, offset + n, dtype=np.int64)
            rel = _rel_positions(spec.mrope_rel, n, self.use_3d)
            own_span = spec.self_prefix_len if spec.self_prefix_span is None else spec.self_prefix_span
            position = own_span + sum(b.mrope_span for b in spec.context)
            for slot, block in enumerate(spec.context):
                assert block.num_tokens > 0, "context blocks must be non-empty"
                i = worker * d + slot
                q_len[i], lengths[i], chain[i] = n, block.num_tokens, worker
                pages[i] = page_numbers_array(block, snapshot)
                gather.append(source)
                slots.append(source * (d + 1) + slot)
                locations.append(rel + position)
                position -= block.mrope_span
            i = w * d + 1 + worker
            q_len[i], lengths[i], chain[i] = n, spec.self_prefix_len + n, worker
            pages[i] = [start // P for start in spec.self_page_starts.cpu().tolist()]
            self_loc[..., offset:offset + n] = rel + own_span
            self_slots[offset:offset + n] = source * (d + 1) + len(spec.context)
            last_rows[worker], offset = offset + n - 1, offset + n
        n_ctx = int(q_len[:w * d].sum())
        q_len[w * d] = self.ctx_rows - n_ctx
        q_len[-1] = r - offset
        kv_counts = np.asarray([len(p) for p in pages], dtype=np.int64)
        n_entries = int(kv_counts.sum())
        if n_entries > self.max_pages:
            raise ValueError("Shared prefill exceeds graph page-index capacity")

        self._wait_for_staging()
        self.refs = []
        if n_entries:
            np.concatenate([np.asarray(part, dtype=np.int32) for part in pages if len(part)],
                           out=self._kv_host.numpy()[:n_entries])
        active = np.concatenate(slots) if slots else np.empty(0, dtype=np.int64)
        unused = np.ones(r * (d + 1), dtype=bool)
        unused[active] = False
        unused[self_slots] = False
        permutation = np.concatenate([active, self._all_slots[unused]])
        assert permutation.size == self.ctx_rows
        sub_worker = self._sub_worker_host.numpy()
        sub_worker[:self.ctx_rows] = 0
        loc = self._loc_host
        loc.zero_()
        if gather:
            sub_worker[:n_ctx] = np.concatenate(gather)
            loc[..., :n_ctx] = torch.cat(locations, dim=-1)
        loc[..., self.ctx_rows:] = self_loc
        valid = self._valid_host.numpy()
        valid[:] = False
        valid[:n_ctx] = True
        valid[self.ctx_rows:self.ctx_rows + offset] = True
        self._pad_host.numpy()[:] = np.concatenate([permutation, self_slots])
        self._last_host.numpy()[:] = last_rows
        qo_indptr = np.concatenate([[0], np.cumsum(q_len)])
        kv_indptr = np.concatenate([[0], np.cumsum(kv_counts)])
        self._build(qo_indptr, kv_indptr, lengths, flags, chain, sub_worker, r)
        for dev, host in ((self.meta.sub_worker, self._sub_worker_host), (self.meta.pad_slot, self._pad_host),
                          (self.meta.last_indices, self._last_host)):
            dev.copy_(host, non_blocking=True)
        if self.event is not None:
            self.event.record()
        self.used_ctx_rows, self.used_self_rows = n_ctx, offset
        self.meta.launch = self._launch()
        return self.meta
