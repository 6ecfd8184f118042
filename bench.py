"""Benchmark of cache-view attention on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME]

A step is one ``SharedCacheAttention.forward`` of one layer (fused key
rotate + KV store, attention, merge).  Without ``--workload`` the line is the
batched bf16 decode configuration (64 requests, 16 q / 4 kv heads, head_dim 256,
page size 16, every view = one shared 8192-token block + 1-3 private blocks of
256..8192 tokens) and carries, under ``configs``, the same measurements for the
view-conditioned prefill, the mixed continuous batch, the long-context mRoPE
decode and the fp32 plumbing case, each measured by a child process of its own
(a fresh allocator and address space, as when the workload is run alone); with
``--workload`` only that workload is measured, in this process.  Inputs are resident in HBM before the timed region; successive steps
rotate over several copies of the KV pool so the 256 MB last-level cache cannot
hold the working set.  Prints ONE JSON line.

``value`` is algorithmic GB/s (decode, mixed) or TFLOP/s (prefill): compulsory
bytes of a step (each distinct block counted once) or flops of the visible
(row, key) pairs, see ``async_llm_amd.workloads``, divided by the wall time per
step.  ``roofline`` prices the attention launches alone, timed with HIP events on
the stream they are launched on.  ``cpu_baseline`` times the CPU oracle (torch on
the host cores) on a bounded sample of the same workload, and ``parity`` compares the
GPU's ``out`` / ``lse`` of that very step with the oracle's outputs for the sample (largest
absolute and relative errors, within tolerance or not) and the planned integer tables of the
whole workload with the oracle's planner, bit for bit; a workload that differs ends the
run with a non-zero exit code.  The region of K timed steps is repeated ``REPEATS`` times;
``ms_per_step`` is the median region and ``ms_per_step_regions`` the fastest and slowest.
"""

from __future__ import annotations

import argparse
import json
import os
import subprocess
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

REPEATS = 5  # timed regions of K steps each; the line reports the median region
HBM_PEAK_GBS = 8000.0
MFMA_BF16_PEAK_TFLOPS = 2500.0

# HBM bytes one launch (attention + merge) moves at the default sizes, from rocprofv3 --pmc
# FETCH_SIZE / WRITE_SIZE runs of this script scaled by the readings of --workload
# copy_calibration (bytes = 2 KiB x FETCH_SIZE + 1 KiB x WRITE_SIZE); the summaries are in
# profiles/.  A counter run cannot be made from inside the timed process, so the figures are
# carried here together with the digest of the kernel sources they were measured on
# (csrc_digest()), and are reported only while that digest is the one of the sources in the tree.
MEASURED_TRAFFIC = {
    ("batched_decode", "mfma"): {"bytes": 2 * 1024 * (1_129_938 + 8_988) + 1024 * (17_885 + 512), "csrc": "08c375c61b54cd3d"},
    ("mrope_decode", "mfma"): {"bytes": 2 * 1024 * (2_098_018 + 4_722) + 1024 * (9_297 + 64), "csrc": "08c375c61b54cd3d"},
    ("view_prefill", "mfma"): {"bytes": 2 * 1024 * 2_496_982 + 1024 * 131_323, "csrc": "08c375c61b54cd3d"},
    ("mixed_batch", "mfma"): {"bytes": 2 * 1024 * (439_645 + 1_623_108 + 27_058) + 1024 * (47_429 + 12_397 + 10_624),
                              "csrc": "08c375c61b54cd3d"},
}


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=None, help="timed steps (default: about a second of GPU time)")
    ap.add_argument("--warmup", type=int, default=None, help="untimed steps before them (default: steps / 10)")
    ap.add_argument("--workload", default=None,
                    choices=["batched_decode", "mrope_decode", "view_prefill", "plumbing_decode", "mixed_batch",
                             "copy_calibration", "block_merge"])
    ap.add_argument("--layers", type=int, default=4, help="copies of the KV pool rotated over")
    ap.add_argument("--kernel", default=None, choices=[None, "auto", "generic", "mfma"])
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--cpu-sample", type=int, default=0, help="requests in the CPU sample (0 = pick by size)")
    return ap.parse_args()


def build_workload(name, device, layers, kernel):
    from async_llm_amd import workloads

    if name == "batched_decode":
        return workloads.batched_decode(device, layers=layers, kernel=kernel)
    if name == "mrope_decode":
        return workloads.mrope_decode(device, layers=layers, kernel=kernel)
    if name == "view_prefill":
        return workloads.view_prefill(device, layers=layers, kernel=kernel)
    if name == "mixed_batch":
        return workloads.mixed_batch(device, layers=layers, kernel=kernel)
    return workloads.plumbing_decode(device, layers=layers, kernel=kernel)


def time_attention_kernel(wl, steps, warmup, layers, repeats=1):
    """Duration of the attention launch alone (store excluded), HIP events recorded on the
    stream the kernels run on, over ``repeats`` regions of ``steps`` launches.  Returns the
    average and the median over all launches and the average of every region."""
    import torch

    op, meta = wl.op, wl.meta
    stream = torch.cuda.current_stream()
    for i in range(warmup):
        op.attend(wl.q, i % layers, meta)
    torch.cuda.synchronize()
    times, region_avg = [], []
    for _ in range(repeats):
        starts = [torch.cuda.Event(enable_timing=True) for _ in range(steps)]
        stops = [torch.cuda.Event(enable_timing=True) for _ in range(steps)]
        for i in range(steps):
            starts[i].record(stream)
            op.attend(wl.q, i % layers, meta)
            stops[i].record(stream)
        torch.cuda.synchronize()
        region = [s.elapsed_time(e) for s, e in zip(starts, stops)]
        region_avg.append(sum(region) / len(region))
        times += region
    times.sort()
    return sum(times) / len(times), times[len(times) // 2], region_avg


def cpu_baseline(wl, sample):
    """The CPU oracle on the first ``sample`` requests of the workload (same
    blocks, same inputs): rotate+store, per-segment attention, merge.  A mixed
    batch takes its first ``sample`` decode rows and its first prefill chunk.
    Returns (seconds per pass, compulsory bytes of the sample, flops of the
    sample, cores, description, timed passes, outputs): ``outputs`` lists, per part of
    the sample, ``(first row, rows, out, lse)`` of the oracle's last pass."""
    import torch

    from async_llm_amd.shared_cache import WorkerGroup
    from oracle import view_attention_oracle as O
    from tests.util import oracle_decode_plan, oracle_prefill_plan, oracle_rope

    op = wl.op
    Hq, Hkv, D, P = op.num_qo_heads, op.num_kv_heads, op.head_dim, op.page_size
    cores = os.cpu_count() or 1
    torch.set_num_threads(cores)
    rope = oracle_rope(op, wl.theta)
    k_cpu, v_cpu = wl.pool.k_cache(0).cpu(), wl.pool.v_cache(0).cpu()
    item = wl.q.element_size()
    b_tok = 2 * Hkv * D * item
    runs, what = [], []
    distinct, pairs = {}, 0
    W = wl.group.num_workers if wl.group is not None else 0
    if wl.mode in ("decode", "mixed"):
        n = min(W, sample)
        group = WorkerGroup(wl.group.workers[:n])
        pending = {id(b): wl.pending[id(b)] for b in group.write_to}
        slots = wl.new_token_slots.cpu()[:n]
        plan = oracle_decode_plan(group, pending, slots, P)
        q, k, v = wl.q.cpu()[:n], wl.k.cpu()[:n], wl.v.cpu()[:n]
        pos = wl.batch.positions.cpu()[:n]
        logical = sum(plan.seq_lens) + len(plan.aux_slots)

        def run_decode():
            k_rot = rope.rotate(k.view(n, Hkv, D), pos)
            O.store_kv(k_cpu.view(-1, Hkv * D), v_cpu.view(-1, Hkv * D), slots, k_rot.reshape(n, -1), v)
            out, lse, _ = O.forward_decode(plan, q.view(n, Hq, D), k_cpu, v_cpu, rope)
            return 0, n, out, lse

        runs.append(run_decode)
        for view in group.cache_structure:  # compulsory bytes of the sample: distinct blocks once
            for b in view:
                distinct[id(b)] = b.num_tokens + (1 if id(b) in pending else 0)
        pairs += logical
        what.append(f"first {n} of {W} decode requests ({logical} logical KV tokens)")
    if wl.mode in ("prefill", "mixed"):
        n_p = min(len(wl.specs), sample if wl.mode == "prefill" else 1)
        specs = wl.specs[:n_p]
        plan_p = oracle_prefill_plan(specs, P)
        rows = plan_p.num_rows
        qp, kp, vp = wl.q.cpu()[W:W + rows], wl.k.cpu()[W:W + rows], wl.v.cpu()[W:W + rows]
        pos_p = wl.batch.positions.cpu()[W:W + rows]
        out_loc = wl.batch.out_loc.cpu()[W:W + rows]

        def run_prefill():
            k_rot = rope.rotate(kp.view(rows, Hkv, D), pos_p)
            O.store_kv(k_cpu.view(-1, Hkv * D), v_cpu.view(-1, Hkv * D), out_loc, k_rot.reshape(rows, -1), vp)
            out, lse = O.forward_prefill_batch(plan_p, qp.view(rows, Hq, D), k_cpu, v_cpu, rope)
            return W, rows, out, lse

        runs.append(run_prefill)
        for s in specs:
            for b in s.context:
                distinct[id(b)] = b.num_tokens
            distinct[("own", id(s))] = s.self_prefix_len + s.num_new
            before = sum(b.num_tokens for b in s.context) + s.self_prefix_len
            pairs += s.num_new * before + s.num_new * (s.num_new + 1) // 2
        what.append(f"first {n_p} of {len(wl.specs)} prefill requests ({rows} new tokens)")

    outputs = []

    def run():
        outputs[:] = [r() for r in runs]

    t0 = time.perf_counter()
    run()
    first = time.perf_counter() - t0
    reps = 3 if first < 4.0 else 1  # a long sample is timed once more after this warm-up pass
    times = []
    for _ in range(reps):
        t0 = time.perf_counter()
        run()
        times.append(time.perf_counter() - t0)
    t = sorted(times)[len(times) // 2]
    sample_bytes = b_tok * sum(distinct.values())
    return t, sample_bytes, 4 * D * Hq * pairs, cores, " + ".join(what), reps, outputs


# out / lse tolerances of the parity contract: 2e-2 abs + 1e-2 rel for 16-bit storage, 1e-5 for fp32
PARITY_TOL = {"bf16": (2e-2, 1e-2), "f16": (2e-2, 1e-2), "f32": (1e-5, 1e-5)}


def index_parity(wl) -> bool:
    """The product's planned integer tables of the WHOLE workload (sub-row owner, rotation
    position, pad slot, page / slot table, segment lengths) against the oracle's planner:
    bit for bit."""
    import torch

    from tests.util import oracle_decode_plan, oracle_prefill_plan

    meta, P = wl.meta, wl.op.page_size
    sub_worker, sub_loc, slot, kv, M = [], [], [], [], meta.max_segments
    checks = []
    W = 0
    if wl.mode in ("decode", "mixed"):
        W = wl.group.num_workers
        d = oracle_decode_plan(wl.group, wl.pending, wl.new_token_slots.cpu(), P)
        sub_worker += d.sub_worker
        loc = torch.tensor(d.sub_loc, dtype=torch.int64)
        sub_loc.append(loc)
        slot += [p - w * d.max_segments for p, w in zip(d.pad_slot, d.sub_worker)]
        kv += d.kv_indices + d.aux_slots
        checks.append((meta.n_main, meta.n_aux) == (d.n_main, d.n_aux))
        if meta.main_plan is not None and wl.mode == "decode":
            checks.append(meta.main_plan["seq_lens"].tolist() == d.seq_lens)
            checks.append(meta.main_plan["last_page_len"].tolist() == d.last_page_len)
            checks.append(meta.main_plan["indptr"].tolist() == d.kv_indptr)
            checks.append(M == d.max_segments)
    if wl.mode in ("prefill", "mixed"):
        p = oracle_prefill_plan(wl.specs, P)
        sub_worker += [r + W for r in p.sub_worker]
        sub_loc.append(p.sub_loc)
        slot += [s - r * p.max_segments for s, r in zip(p.pad_slot, p.sub_worker)]
        kv += p.ctx["kv_indices"] + p.own["kv_indices"]
        checks.append(meta.n_ctx_rows == p.n_ctx_rows)
        checks.append(meta.last_indices.cpu().tolist()[-len(p.last_indices):] == [i + W for i in p.last_indices])
        if wl.mode == "prefill":
            checks.append(meta.main_plan["seq_lens"].tolist() == p.ctx["seq_lens"])
            checks.append(meta.aux_plan["seq_lens"].tolist() == p.own["seq_lens"])
            checks.append(meta.main_plan["paged_kv_last_page_len"].tolist() == p.ctx["last_page_len"])
            checks.append(meta.aux_plan["paged_kv_last_page_len"].tolist() == p.own["last_page_len"])
            checks.append(M == p.max_segments)
    use_3d = any(x.dim() == 2 for x in sub_loc)
    sub_loc = [x if x.dim() == 2 or not use_3d else x.unsqueeze(0).expand(3, -1) for x in sub_loc]
    exp_loc = torch.cat(sub_loc, dim=1 if use_3d else 0)
    exp_worker = torch.tensor(sub_worker, dtype=torch.int64)
    exp_pad = exp_worker * M + torch.tensor(slot, dtype=torch.int64)
    checks.append(torch.equal(meta.sub_worker.cpu(), exp_worker))
    checks.append(torch.equal(meta.sub_loc.cpu(), exp_loc))
    checks.append(torch.equal(meta.pad_slot.cpu(), exp_pad))
    checks.append(meta.launch.kv_indices.cpu().tolist() == kv)
    return all(bool(c) for c in checks)


def parity_block(wl, outputs, dtype_name):
    """Largest errors of the product's ``out`` / ``lse`` (one more step on layer 0, whose pool the
    oracle read) against the oracle's outputs for the rows of the CPU sample."""
    import torch

    out, lse = wl.op.forward_with_lse(wl.q, wl.k, wl.v, 0, wl.batch)
    torch.cuda.synchronize()
    out, lse = out.cpu().double(), lse.cpu().double()
    atol, rtol = PARITY_TOL[dtype_name]
    worst = dict(max_abs_out=0.0, max_rel_out=0.0, max_abs_lse=0.0, max_rel_lse=0.0)
    within, rows_checked = True, 0
    for first, rows, exp_out, exp_lse in outputs:
        for name, got, exp in (("out", out[first:first + rows], exp_out.double()),
                               ("lse", lse[first:first + rows], exp_lse.double())):
            err = (got - exp.reshape(got.shape)).abs()
            ref = exp.reshape(got.shape).abs()
            worst["max_abs_" + name] = max(worst["max_abs_" + name], err.max().item())
            # relative error where the reference is large enough for the ratio to mean something
            big = ref > 10 * atol
            if big.any():
                worst["max_rel_" + name] = max(worst["max_rel_" + name], (err[big] / ref[big]).max().item())
            within = within and bool((err <= atol + rtol * ref).all()) and bool(torch.isfinite(got).all())
        rows_checked += rows
    block = {k: float("%.3e" % v) for k, v in worst.items()}
    block.update(within_tol=within, tolerance={"abs": atol, "rel": rtol}, rows_checked=rows_checked,
                 indices_bit_exact=index_parity(wl))
    return block


def copy_calibration(dev, steps):
    """A plain device copy of known size (1 GiB read + 1 GiB written per launch):
    what the FETCH_SIZE / WRITE_SIZE counters read for it gives the factor that
    turns their readings for the attention kernels into bytes."""
    import torch

    n = 1 << 30
    src = torch.empty(n, dtype=torch.uint8, device=dev).fill_(3)
    dst = torch.empty_like(src)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        dst.copy_(src)
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / steps
    print(json.dumps({"workload": "copy_calibration", "bytes_read": n, "bytes_written": n, "steps": steps,
                      "ms_per_copy": round(ms, 4), "gbps_read_plus_write": round(2 * n / ms / 1e6, 1)}), flush=True)
    return 0


def block_merge(dev, steps, warmup, layers, cpu):
    """Merge of two 16384-token blocks (16 q / 4 kv heads, head_dim 256, bf16, page 16) over
    ``layers`` layers: left copied, right copied with its keys rotated by the left span.  One step =
    the two ``va_copy_shift_kv`` launches of ``BlockKVOps.merge_blocks``; algorithmic bytes =
    4 * layers * kv_heads * head_dim * 2 B per token (K and V, read and written once)."""
    import numpy as np
    import torch

    from async_llm_amd.kvcache.mha_pool import MHAKVCache
    from async_llm_amd.kvcache.page_allocator import PageAllocator
    from async_llm_amd.shared_cache import BlockKVOps, SharedCacheAttention
    from async_llm_amd.shared_cache.block_ops import token_slots

    Hq, Hkv, D, P, n_left, n_right = 16, 4, 256, 16, 16384, 16384
    num_pages = 4 * (n_left + n_right) // P
    pool = MHAKVCache(Hkv, layers, D, num_pages, P, torch.bfloat16, dev)
    pool._kv_buffer.normal_()
    half = D // 2
    inv = 1.0 / (1e6 ** (torch.arange(half, dtype=torch.float32) / half))
    angles = torch.arange(32768, dtype=torch.float32)[:, None] * inv[None, :]
    table = torch.cat([angles.cos(), angles.sin()], dim=-1).to(dev)
    att = SharedCacheAttention(pool, table, Hq, Hkv, D, P, torch.bfloat16, dev)
    allocator = PageAllocator(num_pages, P, dev)
    allocator._free = allocator._free[torch.randperm(num_pages, device=dev)]  # a pool in use: scattered pages
    ops = BlockKVOps(pool, att, allocator)
    left, right = ops.create_block(), ops.create_block()
    left.grow_pages(allocator.alloc_pages(n_left // P), n_left)
    right.grow_pages(allocator.alloc_pages(n_right // P), n_right)
    merged = ops.merge_blocks(left, right)
    torch.cuda.synchronize()
    src_l, src_r, dst = token_slots(left), token_slots(right), token_slots(merged)

    def step():
        ops._launch(src_l, dst[:n_left], 0)
        ops._launch(src_r, dst[n_left:], left.mrope_span)

    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) * 1e3 / steps
    # the launches alone: slot tables already on the device
    tables = torch.from_numpy(np.stack([np.concatenate([src_l, src_r]), dst])).to(dev)
    stream = torch.cuda.current_stream(dev)
    width, stride = Hkv * D, pool.k_cache(1).data_ptr() - pool.k_cache(0).data_ptr() if layers > 1 else 0
    from async_llm_amd import native

    def launches():
        for first, n, shift in ((0, n_left, 0), (n_left, n_right, left.mrope_span)):
            native.check(native.lib.va_copy_shift_kv(
                pool.k_cache(0).data_ptr(), pool.v_cache(0).data_ptr(), width, stride // 2, layers,
                tables[0, first:].data_ptr(), tables[1, first:].data_ptr(), n, shift, att._shape,
                att._rope_descriptor(), stream.cuda_stream))

    times = []
    for i in range(warmup + steps):
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record(stream)
        launches()
        b.record(stream)
        b.synchronize()
        if i >= warmup:
            times.append(a.elapsed_time(b))
    kern_ms = sum(times) / len(times)
    alg_bytes = 4 * layers * Hkv * D * 2 * (n_left + n_right)
    line = {
        "metric": "block_merge_hbm_gbps", "value": round(alg_bytes / ms_per_step / 1e6, 1), "unit": "GB/s",
        "n_gpus": 1, "steps": steps, "warmup": warmup, "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "block_merge", "left_tokens": n_left, "right_tokens": n_right, "layers": layers,
                   "kv_heads": Hkv, "head_dim": D, "page_size": P, "alg_bytes": alg_bytes},
        "roofline": {"bound": "hbm", "achieved": round(alg_bytes / kern_ms / 1e6, 1), "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": round(alg_bytes / kern_ms / 1e6 / HBM_PEAK_GBS, 4), "traffic": None,
                     "kernel": "copy_shift_kernel x2 (left copy, right copy + key shift)",
                     "kernel_ms_avg": round(kern_ms, 4)},
    }
    if cpu:
        from oracle import view_attention_oracle as O

        n = 4096  # tokens of each block in the sample, one layer
        k_cpu = pool.k_cache(0)[: 4 * n // P].cpu().reshape(-1, Hkv, D)
        v_cpu = pool.v_cache(0)[: 4 * n // P].cpu().reshape(-1, Hkv, D)
        rope = O.RopeSpec(D, table.cpu())
        reps = []
        for _ in range(3):
            t0 = time.perf_counter()
            O.copy_shift_kv(k_cpu, v_cpu, range(0, n), range(2 * n, 3 * n), 0, rope)
            O.copy_shift_kv(k_cpu, v_cpu, range(n, 2 * n), range(3 * n, 4 * n), n, rope)
            reps.append(time.perf_counter() - t0)
        t = sorted(reps)[1]
        line["cpu_baseline"] = {"value": round(4 * Hkv * D * 2 * 2 * n / t / 1e9, 3), "unit": "GB/s",
                                "cores": torch.get_num_threads(), "kind": "port",
                                "sample": f"two {n}-token blocks, one layer, {t:.3f} s per pass, torch CPU oracle, "
                                          "median of 3"}
    print(json.dumps(line), flush=True)
    return 0


def cpu_model() -> str:
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.lower().startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def csrc_digest() -> str:
    """Digest of the kernel and planner sources: a traffic figure measured with rocprofv3 is only
    reported while the sources it was measured on are the ones that are running."""
    import hashlib

    h = hashlib.sha256()
    src = os.path.join(ROOT, "async_llm_amd", "csrc")
    for name in sorted(os.listdir(src)):
        with open(os.path.join(src, name), "rb") as f:
            h.update(name.encode() + b"\0" + f.read())
    return h.hexdigest()[:16]


def host_prepare_ms(wl, reps=20):
    """Median wall time of planning the step again on the host (``prepare`` /
    ``prepare_prefill_batch`` / ``prepare_mixed``), uploads included."""
    import torch

    op = wl.op
    if wl.mode == "decode":
        call = lambda: op.prepare(wl.group, wl.pending, wl.new_token_slots)
    elif wl.mode == "prefill":
        call = lambda: op.prepare_prefill_batch(wl.specs)
    else:
        call = lambda: op.prepare_mixed(wl.group, wl.pending, wl.new_token_slots, wl.specs)
    times = []
    for _ in range(reps):
        t0 = time.perf_counter()
        meta = call()
        times.append((time.perf_counter() - t0) * 1e3)
        del meta
    torch.cuda.synchronize()
    return sorted(times)[len(times) // 2]


def measure(wl, steps, warmup, layers, cpu_sample, with_cpu, traffic_ok):
    """Time one workload: whole steps by the wall clock, the attention launches alone with HIP
    events, the host planner, and the CPU oracle on a bounded sample.  Returns the fields of a
    bench line (``steps`` / ``warmup`` as used)."""
    import torch

    # The shader clock idles at ~0.15 GHz and takes some milliseconds of load to reach its working
    # frequency: run the step untimed for a while first (not counted in W or K), so that a short
    # K measures the kernels and not the ramp.
    t_ramp = time.perf_counter()
    while time.perf_counter() - t_ramp < 0.2:
        for i in range(8):
            wl.forward(i % layers)
        torch.cuda.synchronize()
    if steps is None:  # about a second of steps
        t0 = time.perf_counter()
        for i in range(8):
            wl.forward(i % layers)
        torch.cuda.synchronize()
        steps = max(20, min(2000, int(8 / (time.perf_counter() - t0))))
    if warmup is None:
        warmup = max(4, steps // 10)

    # whole step (store + attention + merge), wall clock around K steps; the region of K steps is
    # timed REPEATS times over (a single short region cannot resolve differences of a percent or two:
    # clock and box drift are of that size) and the line carries the median region and the spread
    for i in range(warmup):
        wl.forward(i % layers)
    torch.cuda.synchronize()
    regions = []
    for _ in range(REPEATS):
        t0 = time.perf_counter()
        for i in range(steps):
            wl.forward(i % layers)
        torch.cuda.synchronize()
        regions.append((time.perf_counter() - t0) * 1e3 / steps)
    ms_per_step = sorted(regions)[len(regions) // 2]

    kern_avg_ms, kern_med_ms, kern_regions = time_attention_kernel(wl, steps, warmup, layers, REPEATS)
    counts = wl.meta.launch.counts
    family = {1: "generic", 2: "mfma"}.get(counts.kernel)
    decode = wl.mode in ("decode", "mixed")  # the mixed batch is priced against HBM, its binding roof
    if decode:
        metric, unit = "view_attention_decode_hbm_gbps", "GB/s"
        value = wl.alg_bytes / (ms_per_step * 1e-3) / 1e9
        achieved = wl.alg_bytes / (kern_avg_ms * 1e-3) / 1e9
        roof = dict(bound="hbm", achieved=round(achieved, 1), peak=HBM_PEAK_GBS, unit="GB/s",
                    frac=round(achieved / HBM_PEAK_GBS, 4), traffic=None)
    else:
        metric, unit = "view_attention_prefill_mfma_tflops", "TFLOP/s"
        value = wl.alg_flops / (ms_per_step * 1e-3) / 1e12
        achieved = wl.alg_flops / (kern_avg_ms * 1e-3) / 1e12
        roof = dict(bound="mfma", achieved=round(achieved, 2), peak=MFMA_BF16_PEAK_TFLOPS, unit="TFLOP/s",
                    frac=round(achieved / MFMA_BF16_PEAK_TFLOPS, 4), traffic=None)
    measured = MEASURED_TRAFFIC.get((wl.name, family))
    if traffic_ok and measured and measured["csrc"] == csrc_digest():
        roof["traffic"] = measured["bytes"]
        roof["traffic_source"] = "rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, sources " + measured["csrc"]
    roof.update(kernel="attention launch (all work items) + merge", kernel_ms_avg=round(kern_avg_ms, 4),
                kernel_ms_median=round(kern_med_ms, 4),
                kernel_ms_regions=[round(min(kern_regions), 4), round(max(kern_regions), 4)])
    dtype = (str(wl.op.dtype).replace("torch.", "").replace("bfloat16", "bf16").replace("float32", "f32")
             .replace("float16", "f16"))
    line = {
        "metric": metric, "value": round(value, 2), "unit": unit, "n_gpus": 1, "steps": steps,
        "warmup": warmup, "ms_per_step": round(ms_per_step, 4), "repeats": REPEATS,
        "ms_per_step_regions": [round(min(regions), 4), round(max(regions), 4)],
        "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": dtype, "data": "synthetic",
        "config": {"workload": wl.name, "rows": wl.info.get("rows"), "q_heads": wl.op.num_qo_heads,
                   "kv_heads": wl.op.num_kv_heads, "head_dim": wl.op.head_dim, "page_size": wl.op.page_size,
                   "kv_pool_copies": layers, "alg_bytes": wl.alg_bytes, "logical_bytes": wl.logical_bytes,
                   "alg_flops": wl.alg_flops, "kernel_family": family, "work_items": counts.n_items,
                   "wide_items": counts.n_wide_items, "kv_chunk": counts.kv_chunk, "q_tile": counts.q_tile,
                   "partials": counts.n_partials, "host_prepare_ms": round(host_prepare_ms(wl), 3)},
        "roofline": roof,
    }
    if with_cpu:
        sample = cpu_sample or {"decode": 64, "prefill": 1, "mixed": 8}[wl.mode]
        t_cpu, sample_bytes, sample_flops, cores, what, reps, outputs = cpu_baseline(wl, sample)
        if decode:
            cpu_value, cpu_unit = sample_bytes / t_cpu / 1e9, "GB/s"
        else:
            cpu_value, cpu_unit = sample_flops / t_cpu / 1e12, "TFLOP/s"
        line["cpu_baseline"] = {"value": round(cpu_value, 4), "unit": cpu_unit, "cores": cores,
                                "cpu_model": cpu_model(), "kind": "port",
                                "sample": what + f", {t_cpu:.2f} s per pass, torch CPU oracle, "
                                + ("median of 3" if reps == 3 else "one pass after one warm-up" if reps == 1 else f"{reps} passes")}
        # the oracle's outputs of that sample double as the parity check of this very run
        line["parity"] = parity_block(wl, outputs, dtype)
        line["parity"]["sample"] = what
    return line


SECONDARY = ("mrope_decode", "mixed_batch", "view_prefill", "plumbing_decode")


def main() -> int:
    args = parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: view attention runs on a single MI355X here (no collectives, "
              "no sharding); run with --gpus 1", file=sys.stderr)
        return 2
    import torch

    everything = args.workload is None
    if everything:
        # The default run reports every configuration: the batched decode as the line itself, the
        # others under "configs".  Each is measured by a child process of its own (this one never
        # touches the GPU): a configuration then sees the allocator and the address space of a fresh
        # process, as it does when it is run alone or under the profiler, whatever ran before it.
        if torch.cuda.device_count() < 1:
            print("bench.py needs a GPU", file=sys.stderr)
            return 2
        line = None
        for name in ("batched_decode",) + SECONDARY:
            cmd = [sys.executable, os.path.abspath(__file__), "--workload", name,
                   "--layers", str(1 if name == "plumbing_decode" else args.layers)]
            if args.kernel:
                cmd += ["--kernel", args.kernel]
            if name == "batched_decode":
                steps, warmup = args.steps, args.warmup
                cmd += ["--cpu-sample", str(args.cpu_sample)]
            else:
                steps, warmup = (None if name == "plumbing_decode" else max(20, args.steps or 20)), None
            if steps is not None:
                cmd += ["--steps", str(steps)]
            if warmup is not None:
                cmd += ["--warmup", str(warmup)]
            if args.no_cpu_baseline:
                cmd += ["--no-cpu-baseline"]
            child = subprocess.run(cmd, stdout=subprocess.PIPE, text=True)
            rows = [r for r in child.stdout.splitlines() if r.startswith("{")]
            if child.returncode != 0 or not rows:
                print("bench.py: measuring %s failed (exit code %d)" % (name, child.returncode), file=sys.stderr)
                return child.returncode or 1
            sub = json.loads(rows[-1])
            if line is None:
                line = sub
                line["configs"] = {}
                continue
            line["configs"][name] = {
                "metric": sub["metric"], "value": sub["value"], "unit": sub["unit"], "dtype": sub["dtype"],
                "steps": sub["steps"], "warmup": sub["warmup"], "ms_per_step": sub["ms_per_step"],
                "alg_bytes": sub["config"]["alg_bytes"], "alg_flops": sub["config"]["alg_flops"],
                "rows": sub["config"]["rows"], "work_items": sub["config"]["work_items"],
                "wide_items": sub["config"]["wide_items"], "partials": sub["config"]["partials"],
                "host_prepare_ms": sub["config"]["host_prepare_ms"], "roofline": sub["roofline"],
                "ms_per_step_regions": sub["ms_per_step_regions"], "repeats": sub["repeats"],
                "cpu_baseline": sub.get("cpu_baseline"), "parity": sub.get("parity")}
        print(json.dumps(line), flush=True)
        return 0

    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        return 2
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    if args.workload in ("copy_calibration", "block_merge"):
        args.steps = 40 if args.steps is None else args.steps
        args.warmup = 8 if args.warmup is None else args.warmup
    if args.workload == "copy_calibration":
        return copy_calibration(dev, args.steps)
    if args.workload == "block_merge":
        return block_merge(dev, args.steps, args.warmup, args.layers, not args.no_cpu_baseline)
    # naming a workload measures that one alone, in this process (what the profiler runs do)
    traffic_ok = args.layers == 4 and not os.environ.get("VIEWATTN_PLAN")
    wl = build_workload(args.workload, dev, args.layers, args.kernel)
    line = measure(wl, args.steps, args.warmup, args.layers, args.cpu_sample, not args.no_cpu_baseline, traffic_ok)
    print(json.dumps(line), flush=True)
    parity = line.get("parity")
    if parity and not (parity["within_tol"] and parity["indices_bit_exact"]):
        print("bench.py: %s differs from the oracle: %s" % (args.workload, json.dumps(parity)), file=sys.stderr)
        return 3
    return 0


if __name__ == "__main__":
    sys.exit(main())
