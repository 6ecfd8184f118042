"""Shared helpers of the parity tests: mirror product blocks into the oracle's
plain blocks, and compare tensors with the tolerances of the parity contract."""

from __future__ import annotations

import torch

from oracle import view_attention_oracle as O

# out / lse tolerances: 2e-2 abs + 1e-2 rel for 16-bit storage, 1e-5 for fp32
TOL = {torch.float32: (1e-5, 1e-5), torch.bfloat16: (2e-2, 1e-2), torch.float16: (2e-2, 1e-2)}


def mirror(blocks):
    """``id(product block) -> oracle block`` with the same pages, length, span."""
    return {id(b): O.OBlock(b.page_size, list(b.page_starts), b.num_tokens, b.mrope_span_override) for b in blocks}


def all_blocks(group):
    seen = {}
    for view, target in zip(group.cache_structure, group.write_to):
        for b in list(view) + [target]:
            seen[id(b)] = b
    return list(seen.values())


def oracle_decode_plan(group, pending, slots, page_size):
    m = mirror(all_blocks(group))
    views = [[m[id(b)] for b in view] for view in group.cache_structure]
    targets = [m[id(b)] for b in group.write_to]
    opending = {id(m[key]): val for key, val in pending.items()}
    return O.plan_decode(views, targets, opending, [int(s) for s in slots.tolist()], page_size)


def oracle_prefill_plan(specs, page_size):
    blocks = {}
    for s in specs:
        for b in s.context:
            blocks[id(b)] = b
    m = mirror(blocks.values())
    ospecs = [O.OPrefillSpec([m[id(b)] for b in s.context], [int(x) for x in s.self_page_starts.tolist()], s.num_new,
                             s.self_prefix_len, s.self_prefix_span,
                             None if s.mrope_rel is None else s.mrope_rel.cpu()) for s in specs]
    return O.plan_prefill_batch(ospecs, page_size)


def oracle_rope(op, theta):
    """Oracle rotation matching a product op (table rebuilt on the CPU)."""
    if op.mrope_section is not None:
        return O.RopeSpec(op.rotary_dim, None, tuple(op.mrope_section), O.mrope_inv_freq(op.rotary_dim, theta))
    return O.RopeSpec(op.rotary_dim, op.cos_sin_cache.detach().cpu().float())


def assert_close(actual: torch.Tensor, expected: torch.Tensor, dtype, what: str = ""):
    atol, rtol = TOL[dtype]
    a, e = actual.detach().cpu().double(), expected.detach().cpu().double()
    err = (a - e).abs()
    bound = atol + rtol * e.abs()
    worst = (err - bound).max().item() if err.numel() else -1.0
    assert worst <= 0, f"{what}: max abs err {err.max().item():.3e} exceeds {atol}+{rtol}*|ref| by {worst:.3e}"


# ---------------------------------------------------------------------------
# end-to-end comparisons: product op on the GPU vs the oracle on the CPU
# ---------------------------------------------------------------------------
def make_op_and_pool(device, dtype, heads, page, num_pages, theta, rotary_dim=None, mrope_section=None, seed=0,
                     scale=None, kernel=None, max_pos=4096):
    """Random paged pool (kept on the CPU for the oracle and copied to the GPU
    for the op) and the product op over it."""
    from types import SimpleNamespace

    from async_llm_amd.shared_cache import SharedCacheAttention

    Hq, Hkv, D = heads
    g = torch.Generator().manual_seed(seed)
    scale = D ** -0.5 if scale is None else scale
    k_cpu = (torch.randn(num_pages, page, Hkv, D, generator=g) * scale).to(dtype)
    v_cpu = (torch.randn(num_pages, page, Hkv, D, generator=g) * scale).to(dtype)
    k_dev, v_dev = k_cpu.to(device), v_cpu.to(device)
    pool = SimpleNamespace(k_cache=lambda layer: k_dev, v_cache=lambda layer: v_dev)
    rd = D if rotary_dim is None else rotary_dim
    table = O.build_cos_sin_cache(rd, max_pos, theta)
    op = SharedCacheAttention(pool, table.to(device), Hq, Hkv, D, page, dtype, torch.device(device), rotary_dim=rd,
                              mrope_section=mrope_section, rope_base=theta if mrope_section else None, kernel=kernel)
    return op, (k_cpu, v_cpu), (k_dev, v_dev), g


def fused_rows(dev, *parts):
    """The rows of ``parts`` (CPU tensors ``[N, width_i]``) as column slices of ONE device tensor
    ``[N, sum(width_i) + gap]``, the way an attention layer hands q, k and v to the op: views into
    its fused qkv projection, row stride = the projection's width (reference
    ``layers/attention.py:47-64``)."""
    gap = 64  # unrelated columns, poisoned: a kernel that ignored the row stride would read them
    fused = torch.cat(list(parts) + [torch.full((parts[0].shape[0], gap), float("nan"), dtype=parts[0].dtype)], dim=1).to(dev)
    views, at = [], 0
    for part in parts:
        views.append(fused[:, at:at + part.shape[1]])
        at += part.shape[1]
    assert all(not v.is_contiguous() or v.shape[0] <= 1 for v in views)
    return views


def run_decode_parity(op, cpu_pool, dev_pool, group, page_alloc, theta, gen, scale=None, check_pool_exact=True,
                      lse_base2=False, fused_qkv=False):
    """One decode step through the product op and through the oracle; returns
    the product and oracle outputs after asserting parity.  ``fused_qkv``: q, k and v reach
    the op as row-strided slices of one tensor."""
    from types import SimpleNamespace

    from async_llm_amd.shared_cache.session_planning import plan_decode_writes

    dev = op.device
    Hq, Hkv, D, P = op.num_qo_heads, op.num_kv_heads, op.head_dim, op.page_size
    W = group.num_workers
    scale = D ** -0.5 if scale is None else scale
    pending, slots, write_pos = plan_decode_writes(group, P, page_alloc, dev)
    meta = op.prepare(group, pending, slots)
    oplan = oracle_decode_plan(group, pending, slots.cpu(), P)
    assert meta.sub_loc.tolist() == oplan.sub_loc and meta.pad_slot.tolist() == oplan.pad_slot
    q = (torch.randn(W, Hq * D, generator=gen) * scale).to(op.dtype)
    k = (torch.randn(W, Hkv * D, generator=gen) * scale).to(op.dtype)
    v = (torch.randn(W, Hkv * D, generator=gen) * scale).to(op.dtype)
    positions = torch.tensor(write_pos, dtype=torch.int64)
    batch = SimpleNamespace(attn_metadata=meta, positions=positions.to(dev), out_loc=slots, mrope_positions=None)
    q_dev, k_dev, v_dev = fused_rows(dev, q, k, v) if fused_qkv else (q.to(dev), k.to(dev), v.to(dev))
    out, lse = op.forward_with_lse(q_dev, k_dev, v_dev, 0, batch, lse_base2=lse_base2)
    torch.cuda.synchronize()

    rope = oracle_rope(op, theta)
    k_cpu, v_cpu = cpu_pool
    k_rot = rope.rotate(k.view(W, Hkv, D), positions)
    O.store_kv(k_cpu.view(-1, Hkv * D), v_cpu.view(-1, Hkv * D), slots.cpu(), k_rot.reshape(W, -1), v)
    if check_pool_exact:
        assert torch.equal(dev_pool[1].cpu(), v_cpu), "V pool differs"
        if op.mrope_section is None:
            assert torch.equal(dev_pool[0].cpu(), k_cpu), "K pool differs (rotate+store must be bit-exact)"
        else:
            assert_close(dev_pool[0].cpu().float(), k_cpu.float(), op.dtype, "K pool")
    exp_out, exp_lse, _ = O.forward_decode(oplan, q.view(W, Hq, D), k_cpu, v_cpu, rope)
    if lse_base2:
        exp_lse = exp_lse / 0.6931471805599453
    assert out.shape == (W, Hq * D) and out.dtype == op.dtype
    assert_close(out, exp_out, op.dtype, "out")
    assert_close(lse, exp_lse, op.dtype, "lse")
    return out, lse, exp_out, exp_lse, meta


def prefill_inputs(op, specs, gen, scale=None):
    """Write positions, destination slots and random q/k/v rows (CPU tensors) of a
    batched prefill, request-major: ``(positions, mrope_positions, out_loc, q, k, v)``."""
    Hq, Hkv, D, P = op.num_qo_heads, op.num_kv_heads, op.head_dim, op.page_size
    scale = D ** -0.5 if scale is None else scale
    use_3d = any(s.mrope_rel is not None for s in specs) or op.mrope_section is not None
    positions, mpos, out_loc = [], [], []
    for s in specs:
        T, S = s.self_prefix_len, s.num_new
        span = T if s.self_prefix_span is None else s.self_prefix_span
        starts = s.self_page_starts.cpu().to(torch.int64)
        slots = (starts[:, None] + torch.arange(P)[None, :]).reshape(-1)[T:T + S]
        out_loc.append(slots.to(torch.int32))
        positions.append(torch.arange(T, T + S))
        rel = torch.arange(S).expand(3, -1) if s.mrope_rel is None else s.mrope_rel.cpu()
        mpos.append(rel + span)
    positions = torch.cat(positions)
    mrope_positions = torch.cat(mpos, dim=1) if use_3d else None
    out_loc = torch.cat(out_loc)
    N = positions.numel()
    q = (torch.randn(N, Hq * D, generator=gen) * scale).to(op.dtype)
    k = (torch.randn(N, Hkv * D, generator=gen) * scale).to(op.dtype)
    v = (torch.randn(N, Hkv * D, generator=gen) * scale).to(op.dtype)
    return positions, mrope_positions, out_loc, q, k, v


def oracle_prefill(op, cpu_pool, specs, theta, positions, mrope_positions, out_loc, q, k, v):
    """Store the new rows into the CPU pool and run the oracle's batched prefill."""
    Hq, Hkv, D, P = op.num_qo_heads, op.num_kv_heads, op.head_dim, op.page_size
    N = q.shape[0]
    rope = oracle_rope(op, theta)
    k_cpu, v_cpu = cpu_pool
    key_pos = positions if mrope_positions is None else mrope_positions
    k_rot = rope.rotate(k.view(N, Hkv, D), key_pos)
    O.store_kv(k_cpu.view(-1, Hkv * D), v_cpu.view(-1, Hkv * D), out_loc, k_rot.reshape(N, -1), v)
    return O.forward_prefill_batch(oracle_prefill_plan(specs, P), q.view(N, Hq, D), k_cpu, v_cpu, rope)


def run_prefill_parity(op, cpu_pool, dev_pool, specs, theta, gen, scale=None, mutate=None, fused_qkv=False):
    """One batched prefill through the product op and through the oracle.  ``mutate(q, k, v)`` may
    edit the random input rows (CPU tensors) in place before either side sees them; ``fused_qkv``:
    q, k and v reach the op as row-strided slices of one tensor."""
    from types import SimpleNamespace

    dev = op.device
    Hq, D, P = op.num_qo_heads, op.head_dim, op.page_size
    meta = op.prepare_prefill_batch(specs)
    oplan = oracle_prefill_plan(specs, P)
    assert torch.equal(meta.sub_loc.cpu(), oplan.sub_loc) and meta.pad_slot.tolist() == oplan.pad_slot
    N = meta.num_workers
    positions, mrope_positions, out_loc, q, k, v = prefill_inputs(op, specs, gen, scale)
    if mutate is not None:
        mutate(q, k, v)
    batch = SimpleNamespace(attn_metadata=meta, positions=positions.to(dev), out_loc=out_loc.to(dev),
                            mrope_positions=None if mrope_positions is None else mrope_positions.to(dev))
    q_dev, k_dev, v_dev = fused_rows(dev, q, k, v) if fused_qkv else (q.to(dev), k.to(dev), v.to(dev))
    out, lse = op.forward_with_lse(q_dev, k_dev, v_dev, 0, batch)
    torch.cuda.synchronize()

    exp_out, exp_lse = oracle_prefill(op, cpu_pool, specs, theta, positions, mrope_positions, out_loc, q, k, v)
    k_cpu, v_cpu = cpu_pool
    assert torch.equal(dev_pool[1].cpu(), v_cpu), "V pool differs"
    if op.mrope_section is None:
        assert torch.equal(dev_pool[0].cpu(), k_cpu), "K pool differs"
    else:
        assert_close(dev_pool[0].cpu().float(), k_cpu.float(), op.dtype, "K pool")
    assert out.shape == (N, Hq * D)
    assert_close(out, exp_out, op.dtype, "out")
    assert_close(lse, exp_lse, op.dtype, "lse")
    return out, lse, exp_out, exp_lse, meta
