"""The view-attention kernels as a regular attention backend.

Mirror of the reference's backend interface (``python/minisgl/attention/
base.py:12-43``) and of what its FlashInfer backend does with it
(``attention/fi.py:79-300``): ``prepare_metadata`` turns a batch of requests
(``extend_len`` new tokens each, ``device_len`` tokens of KV, their token slots
in ``page_table[req.table_idx]``) into ragged tables, ``forward`` stores the new
K/V rows and runs causal paged attention over page-size-1 indices, and the
``*_capture`` / ``*_replay`` hooks keep one set of fixed buffers per captured
batch size.  Registered beside the reference's backends
(``attention/__init__.py:20-40``) it keeps plain prefills and decodes, which
carry no cache view, on the HIP path.

Differences from the view path: queries and keys arrive already rotated (the
model's RoPE layer ran), so the kernels run with ``rotary_dim = 0``; every
request is one sub-request over token slots (``VA_SUB_SLOTS``), causal for
prefill; the slot table stays on the device (``torch.cat`` of ``page_table``
rows, as the reference builds it), so the planner is given lengths only.
"""

from __future__ import annotations

from abc import ABC, abstractmethod
from dataclasses import dataclass
from typing import Dict, List, Optional

import numpy as np
import torch

from . import native
from .kvcache.mha_pool import store_rows
from .shared_cache.attention import BaseAttnMetadata, LaunchPlan, SharedCacheAttention


class BaseAttnBackend(ABC):
    """Interface of the reference ``BaseAttnBackend`` (``attention/base.py:18-35``)."""

    @abstractmethod
    def forward(self, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, layer_id: int, batch) -> torch.Tensor: ...

    @abstractmethod
    def prepare_metadata(self, batch) -> None: ...

    @abstractmethod
    def init_capture_graph(self, max_seq_len: int, bs_list: List[int]) -> None: ...

    @abstractmethod
    def prepare_for_capture(self, batch) -> None: ...

    @abstractmethod
    def prepare_for_replay(self, batch) -> None: ...


@dataclass
class ViewAttnMetadata(BaseAttnMetadata):
    """Ragged tables of one batch (fields named as the reference's ``FIMetadata``,
    ``attention/fi.py:46-77``) plus the launch plan."""

    cu_seqlens_q_cpu: torch.Tensor
    cu_seqlens_k_cpu: torch.Tensor
    cu_seqlens_q_gpu: torch.Tensor
    indices: torch.Tensor  # int32 device: token slots of every request, concatenated
    seq_lens_cpu: torch.Tensor
    num_qo_heads: int
    num_kv_heads: int
    head_dim: int
    page_size: int  # 1: the indices are token slots
    dtype: torch.dtype
    sub_worker: torch.Tensor  # int64 device: output row of every query row (the identity)
    sub_loc: torch.Tensor  # int64 device: zeros (nothing is rotated here)
    launch: LaunchPlan
    _refs: tuple = ()

    def get_last_indices(self, bs: int) -> torch.Tensor:
        return self.cu_seqlens_q_gpu[1: 1 + bs] - 1


class _CaptureSlot:
    """Fixed device tables of one captured decode batch size."""

    def __init__(self, backend: "ViewAttnBackend", bs: int, indices: torch.Tensor) -> None:
        op = backend.op
        self.bs = bs
        self.capacity = native.VaPlanCapacity()
        limits = native.VaPlanLimits(bs, bs, 0, 0, 0, bs)
        native.check(native.lib.va_plan_capacity(op._shape, op.plan_params, limits, self.capacity))
        self.words = int(native.lib.va_plan_fixed_words(self.capacity))
        self.blob_host = torch.zeros(self.words, dtype=torch.int32, pin_memory=True)
        self.blob = torch.zeros(self.words, dtype=torch.int32, device=op.device)
        self.indices = indices
        self.counts = native.VaPlanCounts()
        self.header: Optional[np.ndarray] = None
        self.event = torch.cuda.Event()
        self.workspace: Optional[torch.Tensor] = None


class ViewAttnBackend(BaseAttnBackend):
    """``ViewAttnBackend(config, kv_cache, page_table)``: ``config`` offers
    ``num_qo_heads``, ``num_kv_heads`` and ``head_dim`` (already divided by the
    tensor-parallel degree); ``kv_cache`` is the paged pool (``k_cache(layer)``,
    ``v_cache(layer)``, ``device``, ``dtype``); ``page_table`` is the int32
    ``[max_requests, max_seq_len]`` table of token slots on the device."""

    def __init__(self, config, kv_cache, page_table: torch.Tensor, kernel: Optional[str] = None) -> None:
        self.config = config
        self.kvcache = kv_cache
        self.page_table = page_table
        self.device = torch.device(kv_cache.device)
        self.op = SharedCacheAttention(kv_cache, None, config.num_qo_heads, config.num_kv_heads, config.head_dim,
                                       1, kv_cache.dtype, self.device, rotary_dim=0, kernel=kernel)
        # for recorded decode batches
        self.capture_bs: List[int] = []
        self.max_graph_bs = 0
        self.max_seq_len = 0
        self.capture_indices: Optional[torch.Tensor] = None
        self.graph_slots: Dict[int, _CaptureSlot] = {}

    # ------------------------------------------------------------------
    def _tables(self, batch):
        reqs = batch.padded_reqs
        seqlens_q = [int(req.extend_len) for req in reqs]
        seqlens_k = [int(req.device_len) for req in reqs]
        for nq, nk in zip(seqlens_q, seqlens_k):
            if nq > nk:
                raise ValueError(f"a request extends by {nq} tokens but holds only {nk}")
        qo = np.concatenate([[0], np.cumsum(seqlens_q)]).astype(np.int32)
        kv = np.concatenate([[0], np.cumsum(seqlens_k)]).astype(np.int32)
        lens = np.asarray(seqlens_k, dtype=np.int32)
        if max(seqlens_q) == 1:  # decode: one row per request, sees all its tokens (its own included)
            flags = np.full(len(reqs), native.VA_SUB_SLOTS, dtype=np.int32)
            chain = np.full(len(reqs), -1, dtype=np.int32)
        else:  # (extend) prefill: causal over the request's own tokens, the cached prefix fully visible
            flags = np.full(len(reqs), native.VA_SUB_SLOTS | native.VA_SUB_CAUSAL, dtype=np.int32)
            chain = np.arange(len(reqs), dtype=np.int32)
        return qo, kv, lens, flags, chain

    def _subs(self, qo, kv, lens, flags, chain, sub_worker_host):
        n_rows = int(qo[-1])
        subs = native.VaSubRequests(len(lens), n_rows, n_rows, qo.ctypes.data, kv.ctypes.data, None,
                                    lens.ctypes.data, flags.ctypes.data, chain.ctypes.data,
                                    sub_worker_host.ctypes.data)
        subs._keepalive = (qo, kv, lens, flags, chain, sub_worker_host)
        return subs

    def prepare_metadata(self, batch) -> None:
        """Plan the batch (reference ``attention/fi.py:201-240``)."""
        op = self.op
        reqs = batch.padded_reqs
        qo, kv, lens, flags, chain = self._tables(batch)
        n_rows = int(qo[-1])
        sub_worker_host = np.arange(n_rows, dtype=np.int64)
        subs = self._subs(qo, kv, lens, flags, chain, sub_worker_host)
        counts = native.VaPlanCounts()
        scratch = op._plan_scratch
        rc = native.lib.va_plan_build(subs, op._shape, op.plan_params, scratch.ctypes.data, scratch.size, counts)
        if rc == native.VA_ERR_CAPACITY and counts.plan_words > scratch.size:
            scratch = op._plan_scratch = np.empty(2 * counts.plan_words, dtype=np.int32)
            rc = native.lib.va_plan_build(subs, op._shape, op.plan_params, scratch.ctypes.data, scratch.size, counts)
        native.check(rc)
        host = torch.empty(counts.plan_words, dtype=torch.int32, pin_memory=True)
        host.numpy()[:] = scratch[: counts.plan_words]
        blob = host.to(self.device, non_blocking=True)
        indices = torch.cat([self.page_table[req.table_idx, : req.device_len] for req in reqs]).to(torch.int32)
        cu_q = torch.from_numpy(qo)
        cu_q_pinned = cu_q.pin_memory()
        launch = LaunchPlan(host[: native.PLAN_HEADER_WORDS].numpy().copy(), blob, indices, counts,
                            op._ensure_workspace(counts.workspace_bytes))
        batch.attn_metadata = ViewAttnMetadata(
            cu_seqlens_q_cpu=cu_q, cu_seqlens_k_cpu=torch.from_numpy(kv),
            cu_seqlens_q_gpu=cu_q_pinned.to(self.device, non_blocking=True), indices=indices,
            seq_lens_cpu=torch.from_numpy(lens), num_qo_heads=op.num_qo_heads, num_kv_heads=op.num_kv_heads,
            head_dim=op.head_dim, page_size=1, dtype=op.dtype,
            sub_worker=torch.arange(n_rows, dtype=torch.int64, device=self.device),
            sub_loc=torch.zeros(n_rows, dtype=torch.int64, device=self.device), launch=launch,
            _refs=(host, cu_q_pinned))

    def forward(self, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, layer_id: int, batch) -> torch.Tensor:
        """Store the new K/V rows at ``batch.out_loc`` and attend (reference
        ``attention/fi.py:186-199``); ``q``/``k`` are already rotated."""
        meta = batch.attn_metadata
        assert isinstance(meta, ViewAttnMetadata)
        op = self.op
        native.require_device(q, "q")
        store_rows(self.kvcache.k_cache(layer_id), self.kvcache.v_cache(layer_id), batch.out_loc,
                   k.reshape(k.shape[0], -1), v.reshape(v.shape[0], -1))
        Hq, D = op.num_qo_heads, op.head_dim
        n_rows = meta.sub_worker.numel()
        q2 = q.reshape(q.shape[0], Hq * D)
        if q2.stride(-1) != 1:
            q2 = q2.contiguous()
        assert q2.shape[0] >= n_rows and q2.dtype == op.dtype
        out = torch.empty((n_rows, Hq * D), dtype=op.dtype, device=self.device)
        launch = meta.launch
        ws = launch.workspace
        k_pool, v_pool = self.kvcache.k_cache(layer_id), self.kvcache.v_cache(layer_id)
        native.check(native.lib.va_attention(
            q2.data_ptr(), q2.stride(0), k_pool.data_ptr(), v_pool.data_ptr(), op.num_kv_heads * D,
            launch.blob.data_ptr(), launch.header.ctypes.data, launch.kv_indices.data_ptr(),
            meta.sub_worker.data_ptr(), meta.sub_loc.data_ptr(), 0, out.data_ptr(), None, 0,
            None if ws is None else ws.data_ptr(), 0 if ws is None else ws.numel(),
            op._shape, op._rope_descriptor(), native.current_stream_ptr(self.device)))
        return out

    # ------------------------------------------------------------------
    # recorded decode batches
    # ------------------------------------------------------------------
    def init_capture_graph(self, max_seq_len: int, bs_list: List[int]) -> None:
        """Reserve the shared slot table of all recorded batch sizes (reference
        ``attention/fi.py:242-249``)."""
        assert self.capture_indices is None, "Capture already initialized."
        self.max_graph_bs = max(bs_list)
        self.max_seq_len = max_seq_len
        self.capture_bs = sorted(bs_list)
        self.capture_indices = torch.zeros(self.max_graph_bs * max_seq_len, dtype=torch.int32, device=self.device)
        self._sub_worker = torch.arange(self.max_graph_bs, dtype=torch.int64, device=self.device)
        self._sub_loc = torch.zeros(self.max_graph_bs, dtype=torch.int64, device=self.device)
        self._cu_q = torch.arange(self.max_graph_bs + 1, dtype=torch.int32, device=self.device)

    def _plan_fixed(self, batch, slot: _CaptureSlot) -> None:
        """Write the batch's plan and slot table into the fixed buffers of its batch size."""
        op = self.op
        reqs = batch.padded_reqs
        bs = slot.bs
        assert len(reqs) == bs, f"batch of {len(reqs)} requests for a graph of {bs}"
        qo, kv, lens, flags, chain = self._tables(batch)
        if int(qo[-1]) != bs:
            raise ValueError("recorded batches are decode batches: one new token per request")
        if int(lens.max()) > self.max_seq_len:
            raise ValueError("a request is longer than the recorded maximum sequence length")
        subs = self._subs(qo, kv, lens, flags, chain, np.arange(bs, dtype=np.int64))
        slot.event.synchronize()  # the previous plan's copy has left the pinned blob
        rc = native.lib.va_plan_build_fixed(subs, op._shape, op.plan_params, slot.capacity,
                                            slot.blob_host.data_ptr(), slot.words, slot.counts)
        native.check(rc)
        header = slot.blob_host[: native.PLAN_HEADER_WORDS].numpy().copy()
        if slot.header is None:
            slot.header = header
            slot.workspace = op._ensure_workspace(slot.counts.workspace_bytes)
        elif not np.array_equal(header, slot.header):
            raise RuntimeError("fixed-capacity plan changed its launch geometry")
        slot.blob.copy_(slot.blob_host, non_blocking=True)
        slot.event.record()
        indices = torch.cat([self.page_table[req.table_idx, : req.device_len] for req in reqs]).to(torch.int32)
        slot.indices[: indices.numel()].copy_(indices)
        cu_q = torch.from_numpy(qo)
        meta = ViewAttnMetadata(
            cu_seqlens_q_cpu=cu_q, cu_seqlens_k_cpu=torch.from_numpy(kv),
            cu_seqlens_q_gpu=self._cu_q[: bs + 1],
            indices=slot.indices, seq_lens_cpu=torch.from_numpy(lens), num_qo_heads=op.num_qo_heads,
            num_kv_heads=op.num_kv_heads, head_dim=op.head_dim, page_size=1, dtype=op.dtype,
            sub_worker=self._sub_worker[:bs], sub_loc=self._sub_loc[:bs],
            launch=LaunchPlan(slot.header, slot.blob, slot.indices, slot.counts, slot.workspace))
        batch.attn_metadata = meta

    def prepare_for_capture(self, batch) -> None:
        """Create the fixed buffers of ``batch.size`` and plan the batch into them
        (reference ``attention/fi.py:259-279``)."""
        bs = batch.size
        assert bs in self.capture_bs and bs not in self.graph_slots and self.capture_indices is not None
        self.graph_slots[bs] = _CaptureSlot(self, bs, self.capture_indices)
        self._plan_fixed(batch, self.graph_slots[bs])

    def prepare_for_replay(self, batch) -> None:
        """Re-plan into the fixed buffers of the padded batch size (reference
        ``attention/fi.py:281-286``)."""
        bs = batch.padded_size
        assert self.capture_indices is not None and bs in self.graph_slots
        self._plan_fixed(batch, self.graph_slots[bs])


def create_viewattn_backend(config, kv_cache=None, page_table=None) -> ViewAttnBackend:
    """Factory for the reference's registry (``attention/__init__.py:20-40``).  With
    the reference's global context in reach the pool and the page table come from
    there, as for its own backends."""
    if kv_cache is None or page_table is None:
        from minisgl.core import get_global_ctx  # the host framework, when this runs inside it

        ctx = get_global_ctx()
        kv_cache = ctx.kv_cache if kv_cache is None else kv_cache
        page_table = ctx.page_table if page_table is None else page_table
    return ViewAttnBackend(config, kv_cache, page_table)


def register(registry, name: str = "viewattn") -> None:
    """``register(SUPPORTED_ATTENTION_BACKENDS)`` adds this backend under ``name``."""
    registry.register(name)(create_viewattn_backend)
