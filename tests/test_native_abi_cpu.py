"""The C-ABI library without a GPU: it loads, exports every symbol the header
declares, and its host-side work decomposition covers every (query sub-row,
visible key) pair exactly once with consistent merge lists."""

import ctypes
import os
import random
import re

import numpy as np
import pytest

from async_llm_amd import native

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
H = dict(MAGIC=0, KERNEL=1, Q_TILE=2, KV_CHUNK=3, N_ITEMS=4, N_LINKS=5, N_QREFS=6, N_PARTIALS=7, N_ROW_PARTS=8,
         N_ROWS=9, OFF_ITEMS=10, OFF_LINKS=11, OFF_QREFS=12, OFF_ROW_INDPTR=13, OFF_ROW_IDS=14, OFF_ROW_FLAGS=15,
         N_EMPTY=16, N_SUBROWS=17, N_WIDE=18, WIDE_TILE=19, OFF_QREF_ROWS=20, N_WIDE_SLOTS=21, OFF_WIDE_SLOTS=22,
         MERGE_WAVES=23)
NO_CAUSAL = 0x3FFFFFFF


def test_library_exports_every_declared_symbol():
    with open(os.path.join(ROOT, "include", "viewattn.h")) as f:
        declared = re.findall(r"^VA_API\s+[\w\s\*]+?\b(va_\w+)\s*\(", f.read(), flags=re.M)
    assert sorted(declared) == sorted(native.EXPORTED_SYMBOLS)
    lib = ctypes.CDLL(native.LIB_PATH)
    for name in declared:
        assert getattr(lib, name) is not None
    assert native.lib.va_version() >= 1
    with open(os.path.join(ROOT, "async_llm_amd", "csrc", "va_plan.h")) as f:
        assert int(re.search(r"VA_PLAN_HEADER_WORDS (\d+)", f.read()).group(1)) == native.PLAN_HEADER_WORDS


def build_plan(qo, kvp, kvi, lens, flags, chain, sub_worker, n_rows, heads=(8, 2, 64), page=4, dtype=native.VA_F32,
               kernel=native.VA_KERNEL_GENERIC, q_tile=0, kv_chunk=0, target=0, wide_tile=0):
    arr = [np.ascontiguousarray(a, dtype=np.int32) for a in (qo, kvp, kvi, lens, flags, chain)]
    sw = np.ascontiguousarray(sub_worker, dtype=np.int64)
    subs = native.VaSubRequests(len(lens), len(sw), n_rows, arr[0].ctypes.data, arr[1].ctypes.data,
                                arr[2].ctypes.data if arr[2].size else None, arr[3].ctypes.data,
                                arr[4].ctypes.data, arr[5].ctypes.data, sw.ctypes.data if sw.size else None)
    shape = native.VaShape(heads[0], heads[1], heads[2], page, dtype)
    params = native.VaPlanParams(kernel, q_tile, kv_chunk, target, wide_tile)
    counts = native.VaPlanCounts()
    rc = native.lib.va_plan_count(subs, shape, params, counts)
    if rc:
        return rc, None, None
    blob = np.zeros(counts.plan_words, dtype=np.int32)
    rc = native.lib.va_plan_build(subs, shape, params, blob.ctypes.data, blob.size, counts)
    return rc, blob, counts


def decode_plan(blob):
    h = blob[: native.PLAN_HEADER_WORDS]
    assert h[H["MAGIC"]] == 0x56415031
    items = blob[h[H["OFF_ITEMS"]]: h[H["OFF_ITEMS"]] + 16 * h[H["N_ITEMS"]]].reshape(-1, 16)
    links = blob[h[H["OFF_LINKS"]]: h[H["OFF_LINKS"]] + 8 * h[H["N_LINKS"]]].reshape(-1, 8)
    qrefs = blob[h[H["OFF_QREFS"]]: h[H["OFF_QREFS"]] + h[H["N_QREFS"]]]
    n_rows = h[H["N_ROWS"]]
    indptr = blob[h[H["OFF_ROW_INDPTR"]]: h[H["OFF_ROW_INDPTR"]] + n_rows + 1]
    ids = blob[h[H["OFF_ROW_IDS"]]: h[H["OFF_ROW_IDS"]] + h[H["N_ROW_PARTS"]]]
    flags = blob[h[H["OFF_ROW_FLAGS"]]: h[H["OFF_ROW_FLAGS"]] + n_rows]
    return h, items, links, qrefs, indptr, ids, flags


def check_coverage(blob, qo, kvp, lens, flags, sub_worker, n_rows, fixed=False):
    """Every visible (sub-row, token) is walked exactly once; partial slots and
    row lists are consistent.  ``fixed``: the plan is padded to a capacity, so
    its header holds upper bounds where a packed plan holds counts."""
    h, items, links, qrefs, indptr, ids, rflags = decode_plan(blob)
    sub_of_row = {}
    for s in range(len(lens)):
        for r in range(qo[s], qo[s + 1]):
            sub_of_row[r] = s
    kv_begin_to_sub = {}
    seen = {}
    part_owner = {}
    contributions = [0] * n_rows
    # each class (wide first, then narrow) is padded to a multiple of the 8 dies
    assert h[H["N_WIDE"]] % 8 == 0 and h[H["N_ITEMS"]] % 8 == 0
    assert all(it[5] == 1 for it in items[: h[H["N_WIDE"]]]) and all(it[5] == 0 for it in items[h[H["N_WIDE"]]:])
    # the wide launch runs one workgroup per slot: the slots partition the real wide items, in order
    slots = blob[h[H["OFF_WIDE_SLOTS"]]: h[H["OFF_WIDE_SLOTS"]] + h[H["N_WIDE_SLOTS"]] + 1]
    assert h[H["N_WIDE_SLOTS"]] % 8 == 0 and slots[0] == 0 and all(a <= b for a, b in zip(slots, slots[1:]))
    # waves per merge workgroup: by the states per row, one wave when the rows are many
    n_rows_h, per_row = max(1, int(h[H["N_ROWS"]])), int(h[H["N_ROW_PARTS"]]) // max(1, int(h[H["N_ROWS"]]))
    assert h[H["MERGE_WAVES"]] in (1, 4, 8, 16)
    assert (h[H["MERGE_WAVES"]] == 16) == (per_row >= 48) or h[H["MERGE_WAVES"]] == 1
    assert slots[-1] <= h[H["N_WIDE"]] and all(it[2] == 0 for it in items[slots[-1]: h[H["N_WIDE"]]])
    for it in items:
        lb, nl, nq, part_base = it[0], it[1], it[2], it[3]
        if nq == 0:  # padding item
            assert nl == 0 and part_base == -1
            continue
        assert nl >= 1 and 1 <= nq <= max(h[H["Q_TILE"]], h[H["WIDE_TILE"]])
        assert it[5] == int(nq > h[H["Q_TILE"]])  # kind: wide iff more rows than the narrow tile
        assert list(it[8:14]) == list(links[lb][:6])  # the item carries a copy of its first link
        rows_of_item = None
        for l in links[lb: lb + nl]:
            kv_begin, t0, t1, qref, cbase, lflags = l[:6]
            assert 0 <= t0 < t1
            rows = []
            for i in range(nq):
                sr = int(qrefs[qref + i]) if lflags & 1 else int(qref + i)
                if lflags & 1:  # the row of an indirect entry is stored beside it
                    assert blob[h[H["OFF_QREF_ROWS"]] + qref + i] == sub_worker[sr]
                s = sub_of_row[sr]
                assert kvp[s] == kv_begin or lens[s] == lens[[x for x in range(len(lens)) if kvp[x] == kv_begin][0]]
                assert t1 <= lens[s]
                assert bool(lflags & 2) == bool(flags[s] & 2)
                causal = bool(flags[s] & 1)
                nq_s = qo[s + 1] - qo[s]
                for t in range(t0, t1):
                    visible = (t <= cbase + i) if cbase != NO_CAUSAL else True
                    if causal:
                        local = sr - qo[s]
                        assert cbase != NO_CAUSAL
                        assert (t <= cbase + i) == (t <= lens[s] - nq_s + local)
                    if visible:
                        key = (sr, t)
                        seen[key] = seen.get(key, 0) + 1
                rows.append(int(sub_worker[sr]))
            if rows_of_item is None:
                rows_of_item = rows
            assert rows == rows_of_item  # all links of an item serve the same output rows
        for i, r in enumerate(rows_of_item):
            contributions[r] += 1
            if part_base >= 0:
                assert part_base + i not in part_owner
                part_owner[part_base + i] = r
    for s in range(len(lens)):
        nq_s = qo[s + 1] - qo[s]
        for local in range(nq_s):
            sr = qo[s] + local
            limit = lens[s] - nq_s + local + 1 if flags[s] & 1 else lens[s]
            for t in range(limit):
                assert seen.get((sr, t), 0) == 1, (s, sr, t, seen.get((sr, t), 0))
    assert sum(seen.values()) == len(seen)
    assert sorted(part_owner) == list(range(len(part_owner)))
    assert len(part_owner) <= h[H["N_PARTIALS"]] if fixed else len(part_owner) == h[H["N_PARTIALS"]]
    for r in range(n_rows):
        mine = sorted(int(x) for x in ids[indptr[r]: indptr[r + 1]])
        assert mine == sorted(p for p, owner in part_owner.items() if owner == r)
        if contributions[r] == 0:
            assert rflags[r] == 2
        elif not mine:
            assert rflags[r] == 1 and contributions[r] == 1
        else:
            assert rflags[r] == 0 and len(mine) == contributions[r]
    if not fixed:
        assert h[H["N_EMPTY"]] == sum(1 for r in range(n_rows) if contributions[r] == 0)


def random_tables(rng, page, prefill):
    qo, kvp, kvi, lens, flags, chain, sub_worker = [0], [0], [], [], [], [], []
    n_rows = 0
    shared_pages = [rng.randrange(1000) for _ in range(150)]
    if prefill:
        for r in range(rng.randint(1, 3)):
            S = rng.randint(1, 70)
            rows = list(range(n_rows, n_rows + S))
            n_rows += S
            for j in range(rng.randint(0, 3)):
                L = rng.randint(1, 300)
                npg = -(-L // page)
                kvi += [rng.randrange(1000) for _ in range(npg)]
                kvp.append(len(kvi)); lens.append(L); flags.append(0); chain.append(r)
                sub_worker += rows; qo.append(len(sub_worker))
            T = rng.randint(0, 40)
            npg = -(-(T + S) // page)
            kvi += [rng.randrange(1000) for _ in range(npg)]
            kvp.append(len(kvi)); lens.append(T + S); flags.append(1); chain.append(r)
            sub_worker += rows; qo.append(len(sub_worker))
    else:
        W = rng.randint(1, 9)
        n_rows = W + rng.randint(0, 2)  # trailing rows nobody serves
        for w in range(W):
            for j in range(rng.randint(0, 3)):
                if rng.random() < 0.5:
                    L = 150
                    pages = shared_pages[: -(-L // page)]
                else:
                    L = rng.randint(1, 700)
                    pages = [rng.randrange(1000) for _ in range(-(-L // page))]
                kvi += pages
                kvp.append(len(kvi)); lens.append(L); flags.append(0); chain.append(-1)
                sub_worker.append(w); qo.append(len(sub_worker))
            if rng.random() < 0.4:
                kvi.append(rng.randrange(16000))
                kvp.append(len(kvi)); lens.append(1); flags.append(2); chain.append(-1)
                sub_worker.append(w); qo.append(len(sub_worker))
    return qo, kvp, kvi, lens, flags, chain, sub_worker, n_rows


@pytest.mark.parametrize("seed", range(8))
@pytest.mark.parametrize("prefill", [False, True])
@pytest.mark.parametrize("q_tile,kv_chunk,target", [(0, 0, 0), (4, 64, 0), (3, 128, 4), (16, 0, 1000)])
def test_plan_covers_every_visible_pair_once(seed, prefill, q_tile, kv_chunk, target):
    rng = random.Random(seed * 2 + int(prefill))
    page = rng.choice([1, 4, 16])
    qo, kvp, kvi, lens, flags, chain, sub_worker, n_rows = random_tables(rng, page, prefill)
    rc, blob, counts = build_plan(qo, kvp, kvi, lens, flags, chain, sub_worker, n_rows, page=page, q_tile=q_tile,
                                  kv_chunk=kv_chunk, target=target)
    assert rc == 0, native.lib.va_last_error()
    assert counts.plan_words == blob.size
    assert counts.workspace_bytes == counts.n_partials * 8 * (64 + 2) * 4
    check_coverage(blob, qo, kvp, lens, flags, sub_worker, n_rows)


@pytest.mark.parametrize("seed", range(6))
@pytest.mark.parametrize("prefill", [False, True])
@pytest.mark.parametrize("wide_tile", [0, 8, -1])
def test_matrix_core_plans_with_wide_tiles_cover_every_pair_once(seed, prefill, wide_tile):
    rng = random.Random(100 + seed * 2 + int(prefill))
    page = rng.choice([1, 4, 16])
    qo, kvp, kvi, lens, flags, chain, sub_worker, n_rows = random_tables(rng, page, prefill)
    rc, blob, counts = build_plan(qo, kvp, kvi, lens, flags, chain, sub_worker, n_rows, page=page, dtype=native.VA_BF16,
                                  kernel=native.VA_KERNEL_MFMA, wide_tile=wide_tile, kv_chunk=rng.choice([0, 64]))
    assert rc == 0, native.lib.va_last_error()
    assert counts.kernel == native.VA_KERNEL_MFMA and counts.q_tile == 4
    assert counts.wide_tile == {0: 64, 8: 8, -1: 0}[wide_tile]
    h, items, *_ = decode_plan(blob)
    kinds = [int(i[5]) for i in items]
    assert kinds == sorted(kinds, reverse=True) and sum(kinds) == counts.n_wide_items == h[H["N_WIDE"]]
    if wide_tile < 0:
        assert counts.n_wide_items == 0
    check_coverage(blob, qo, kvp, lens, flags, sub_worker, n_rows)


def test_readers_of_one_block_share_a_tile():
    page, L = 4, 300
    pages = list(range(75))
    qo, kvp, kvi, lens, flags, chain, sw = [0], [0], [], [], [], [], []
    for w in range(6):
        kvi += pages
        kvp.append(len(kvi)); lens.append(L); flags.append(0); chain.append(-1); sw.append(w); qo.append(len(sw))
    rc, blob, counts = build_plan(qo, kvp, kvi, lens, flags, chain, sw, 6, page=page, q_tile=4, kv_chunk=1024)
    assert rc == 0
    h, items, links, qrefs, *_ = decode_plan(blob)
    # 6 readers -> tiles of 4 and 2 rows; the run is one chunk, cut in two (192 + 108 tokens)
    assert sorted((int(i[2]), int(i[4])) for i in items if i[2]) == [(2, 108), (2, 192), (4, 108), (4, 192)]
    check_coverage(blob, qo, kvp, lens, flags, sw, 6)


def test_tiles_of_one_chunk_run_on_one_die():
    """Workgroup b of a launch runs on die b % 8 (each die has its own L2): the tiles
    that stream the same chunk of a shared block sit at consecutive slots of ONE die,
    and the dies carry about the same load."""
    page, L = 16, 2048
    shared = list(range(L // page))
    qo, kvp, kvi, lens, flags, chain, sw = [0], [0], [], [], [], [], []
    n_req = 24
    for w in range(n_req):  # every request reads the shared block ...
        kvi += shared
        kvp.append(len(kvi)); lens.append(L); flags.append(0); chain.append(-1); sw.append(w); qo.append(len(sw))
    rng = random.Random(5)
    for w in range(n_req):  # ... and a private one
        n = rng.randint(100, 1500)
        kvi += [1000 + 100 * w + i for i in range(-(-n // page))]
        kvp.append(len(kvi)); lens.append(n); flags.append(0); chain.append(-1); sw.append(w); qo.append(len(sw))
    rc, blob, counts = build_plan(qo, kvp, kvi, lens, flags, chain, sw, n_req, page=page, q_tile=4, kv_chunk=256)
    assert rc == 0
    h, items, links, *_ = decode_plan(blob)
    assert h[H["N_WIDE"]] == 0
    where = {}
    load = [0] * 8
    for pos, it in enumerate(items):
        if it[2] == 0:
            continue
        l = links[it[0]]
        load[pos % 8] += int(it[4])
        if l[0] == 0:  # kv_begin of the shared block's representative
            where.setdefault(int(l[1]), []).append(pos)
    # 8 chunks of 256 tokens, the last one cut in two
    assert len(where) == L // 256 + 1 and all(len(v) == n_req // 4 for v in where.values())
    for t0, positions in where.items():
        assert len({p % 8 for p in positions}) == 1, (t0, positions)
        slots = sorted(p // 8 for p in positions)
        assert slots == list(range(slots[0], slots[0] + len(slots)))
    assert max(load) <= 1.25 * (sum(load) / 8) + 256
    check_coverage(blob, qo, kvp, lens, flags, sw, n_req)


def test_runs_that_one_tile_reads_are_flagged_read_once():
    """Ten requests read one 4096-token block and own a private block each (bf16, 16 q / 4 kv heads: 4 requests
    fill a 16-row tile).  The shared block is walked by three query tiles, which should find it in the die's
    L2, so its links stay plain; a private block is read by exactly one tile and streams through the caches
    once: its links carry the read-once flag (the streaming kernel then requests the rows non-temporally),
    whether the run is cut into chunks or not."""
    page, shared_len = 16, 4096
    shared_pages = list(range(shared_len // page))
    kvi, kvp, lens, sw = [], [0], [], []
    next_page = len(shared_pages)
    private_len = [700, 64, 3000, 1, 16, 900, 2048, 333, 5000, 50]
    for w, n in enumerate(private_len):
        kvi += shared_pages; kvp.append(len(kvi)); lens.append(shared_len); sw.append(w)
        pages = -(-n // page)
        kvi += list(range(next_page, next_page + pages)); next_page += pages
        kvp.append(len(kvi)); lens.append(n); sw.append(w)
    n_sub = len(lens)
    rc, blob, counts = build_plan(list(range(n_sub + 1)), kvp, kvi, lens, [0] * n_sub, [-1] * n_sub, sw, len(private_len),
                                  heads=(16, 4, 256), page=page, dtype=native.VA_BF16, kernel=native.VA_KERNEL_MFMA)
    assert rc == 0
    check_coverage(blob, list(range(n_sub + 1)), kvp, lens, [0] * n_sub, sw, len(private_len))
    h, items, links, *_ = decode_plan(blob)
    ONCE = 4
    seen = {True: 0, False: 0}
    for it in items:
        if not it[2]:
            continue
        for l in links[it[0]: it[0] + it[1]]:
            is_shared = int(l[0]) in [kvp[2 * w] for w in range(len(private_len))] and int(l[2]) - int(l[1]) > 0 and \
                kvi[int(l[0])] == 0
            assert bool(int(l[5]) & ONCE) == (not is_shared), (list(l), is_shared)
            seen[is_shared] += 1
            # the copy of the first link that travels in the item carries the same flags
            assert int(it[8 + 5]) == int(links[it[0]][5])
    assert seen[True] >= 3 and seen[False] >= len(private_len)


def _shared_block_plan(readers, shared_len, wide_tile=0):
    """`readers` requests over one shared block plus a private block each (bf16, 16 q / 4 kv heads, head_dim 256)."""
    page = 16
    shared_pages = list(range(-(-shared_len // page)))
    kvi, kvp, lens, sw = [], [0], [], []
    next_page = len(shared_pages)
    for w in range(readers):
        kvi += shared_pages; kvp.append(len(kvi)); lens.append(shared_len); sw.append(w)
        n = 300 + 37 * w
        kvi += list(range(next_page, next_page + -(-n // page))); next_page += -(-n // page)
        kvp.append(len(kvi)); lens.append(n); sw.append(w)
    n_sub = len(lens)
    tables = (list(range(n_sub + 1)), kvp, lens, [0] * n_sub, sw, readers)
    rc, blob, counts = build_plan(tables[0], kvp, kvi, lens, [0] * n_sub, [-1] * n_sub, sw, readers, heads=(16, 4, 256),
                                  page=page, dtype=native.VA_BF16, kernel=native.VA_KERNEL_MFMA, wide_tile=wide_tile)
    assert rc == 0, native.lib.va_last_error()
    return blob, counts, tables


def test_many_readers_of_a_long_block_get_wide_tiles_without_being_asked():
    """Narrow tiles (4 requests) stream a block once per tile; wide ones (32 requests) an eighth as often, in a
    launch of their own.  The planner takes them by itself only where the re-reads saved outweigh that launch:
    64 readers x 8192 tokens (14 re-reads of 32 MB) stay narrow, 64 x 32768 and 128 x 8192 go wide; private
    blocks (one reader) never do, a request for no wide tiles is honoured, and every pair is still covered once."""
    for readers, shared_len, want_wide in [(64, 8192, False), (64, 32768, True), (128, 8192, True), (3, 65536, False)]:
        blob, counts, tables = _shared_block_plan(readers, shared_len)
        h, items, links, *_ = decode_plan(blob)
        assert (counts.n_wide_items > 0) == want_wide, (readers, shared_len, counts.n_wide_items)
        for it in items:
            if it[2] and it[5]:  # a wide item: more than 4 requests, all on the shared block
                assert int(it[2]) > 4 and all(int(l[0]) in tables[1][0::2] for l in links[it[0]: it[0] + it[1]])
        check_coverage(blob, *tables)
    blob, counts, tables = _shared_block_plan(64, 32768, wide_tile=-1)
    assert counts.n_wide_items == 0
    blob, counts, tables = _shared_block_plan(64, 8192, wide_tile=32)  # and on request always
    assert counts.n_wide_items > 0
    check_coverage(blob, *tables)


def test_plan_rejects_inconsistent_tables():
    ok = dict(qo=[0, 1], kvp=[0, 2], kvi=[3, 4], lens=[8], flags=[0], chain=[-1], sub_worker=[0], n_rows=1)

    def attempt(**kw):
        args = dict(ok, **kw)
        rc, _, _ = build_plan(args["qo"], args["kvp"], args["kvi"], args["lens"], args["flags"], args["chain"],
                              args["sub_worker"], args["n_rows"], page=4)
        return rc, native.lib.va_last_error().decode()

    assert attempt()[0] == 0
    rc, msg = attempt(lens=[9])
    assert rc == -1 and "does not fit" in msg
    rc, msg = attempt(sub_worker=[5])
    assert rc == -1 and "outside" in msg
    rc, msg = attempt(flags=[1])
    assert rc == -1 and "chain" in msg
    rc, msg = attempt(qo=[0, 2])
    assert rc == -1
    # capacity error from the builder
    arr = build_plan(ok["qo"], ok["kvp"], ok["kvi"], ok["lens"], ok["flags"], ok["chain"], ok["sub_worker"], 1, page=4)
    assert arr[0] == 0
    subs_blob = np.zeros(4, dtype=np.int32)
    a = [np.ascontiguousarray(x, dtype=np.int32) for x in (ok["qo"], ok["kvp"], ok["kvi"], ok["lens"], ok["flags"], ok["chain"])]
    sw = np.ascontiguousarray(ok["sub_worker"], dtype=np.int64)
    subs = native.VaSubRequests(1, 1, 1, a[0].ctypes.data, a[1].ctypes.data, a[2].ctypes.data, a[3].ctypes.data,
                                a[4].ctypes.data, a[5].ctypes.data, sw.ctypes.data)
    rc = native.lib.va_plan_build(subs, native.VaShape(8, 2, 64, 4, 0), native.VaPlanParams(1, 0, 0, 0, 0),
                                  subs_blob.ctypes.data, 4, None)
    assert rc == -2 and "words" in native.lib.va_last_error().decode()


def test_compute_entry_points_refuse_cpu_tensors():
    import torch
    from async_llm_amd.shared_cache import apply_rope_correction

    with pytest.raises(native.ViewAttnError, match="GPU only"):
        apply_rope_correction(torch.zeros(2, 1, 8), torch.zeros(2, dtype=torch.int64), torch.zeros(4, 8))


def _packed_slot_loads(chunk_tokens, views, coverage=True):
    """Plan prefill chunks of `chunk_tokens` new tokens, one per entry of `views` (the lengths of the
    context segments of the chunk's view; its own block holds 100 tokens before the chunk), at
    16 q / 4 kv heads of 256 dims.  Returns (counts, total tokens walked, per-slot loads, per-slot walks):
    a slot's load is the tokens it walks plus the set-up of every (piece, segment) it holds, worth ~640
    tokens; its walk is the list of (first kv entry, first token, last token) of its links in order."""
    page = 16
    qo, kvp, kvi, lens, flags, chain, sw = [0], [0], [], [], [], [], []
    n_rows = 0
    for r, segments in enumerate(views):
        rows = list(range(n_rows, n_rows + chunk_tokens))
        n_rows += chunk_tokens
        for L in segments:
            kvi += list(range(len(kvi), len(kvi) + -(-L // page)))
            kvp.append(len(kvi)); lens.append(L); flags.append(0); chain.append(r)
            sw += rows; qo.append(len(sw))
        kvi += list(range(len(kvi), len(kvi) + -(-(100 + chunk_tokens) // page)))
        kvp.append(len(kvi)); lens.append(100 + chunk_tokens); flags.append(1); chain.append(r)
        sw += rows; qo.append(len(sw))
    rc, blob, counts = build_plan(qo, kvp, kvi, lens, flags, chain, sw, n_rows, heads=(16, 4, 256), page=page,
                                  dtype=native.VA_BF16, kernel=native.VA_KERNEL_MFMA)
    assert rc == 0
    if coverage:  # (every visible pair once: a check of rows x tokens steps in Python)
        check_coverage(blob, qo, kvp, lens, flags, sw, n_rows)
    h, items, links, *_ = decode_plan(blob)
    slots = blob[h[H["OFF_WIDE_SLOTS"]]: h[H["OFF_WIDE_SLOTS"]] + h[H["N_WIDE_SLOTS"]] + 1]
    assert counts.n_wide_slots == h[H["N_WIDE_SLOTS"]] == 64 and counts.n_wide_items >= 64
    loads = [int(items[a:b, 4].sum()) + 640 * int(items[a:b, 1].sum()) for a, b in zip(slots, slots[1:])]
    # no piece too small to be worth a set-up of its own: at least ~384 tokens + a segment's 640, unless
    # the slots themselves are so small that a remainder of that size would unbalance them (an eighth of a slot)
    assert min(int(it[4]) + 640 * int(it[1]) for it in items[: slots[-1]]) >= min(384 + 640, sum(loads) // 64 // 8) - 16
    walks = [[tuple(int(x) for x in l[:3]) for it in items[a:b] for l in links[it[0]: it[0] + it[1]]]
             for a, b in zip(slots, slots[1:])]
    return counts, int(items[: slots[-1], 4].sum()), loads, walks


def test_few_wide_tiles_are_packed_into_slots_of_equal_length():
    """Prefill chunks whose wide tiles (32 tokens x 4 heads each) cannot fill 64 workgroup slots per
    kv head evenly: views of 1.5k to 30k tokens, and cut one by one into similar pieces the tiles
    would still fill the slots unevenly.  The planner bundles the tiles of a chunk (they walk the
    same view), lays the bundles' walks end to end and gives every group of eight slots -- the
    slots of one die, which walk a bundle side by side -- the same share, set-ups included; a group
    holds the end of one bundle and the start of the next.  The longest slot is the time of the
    launch (one workgroup per CU, one round): it must stay close to the mean, and no slot may be
    left to take a long remainder."""
    # 8 tiles for 64 slots: two tiles a chunk, so a bundle walks four quarters of its view side by side.
    # A group's share is ~3000 tokens here, of which a set-up is a fifth and the least piece a third:
    # that is the grain the groups can be equal to.
    counts, total, loads, _ = _packed_slot_loads(64, [(512, 30000), (512, 1500), (512, 12345), (512, 22222)])
    assert total == 2 * (4 * 512 + 30000 + 1500 + 12345 + 22222) + sum(2 * 100 + 32 + 64 for _ in range(4))
    # the longest slot is the time of the launch; slots at the end may be short or empty
    assert sum(loads) >= 0.84 * 64 * max(loads), (min(loads), max(loads), sum(loads) / 64)
    # 64 tiles for 64 slots (four chunks of 512 tokens over views of two to five blocks: two bundles of eight
    # tiles a chunk): most groups hold the end of one bundle and the start of the next
    views = [(512, 9000, 14000), (512, 2500), (512, 7000, 8000, 9000, 6000), (512, 900, 11000, 3000)]
    counts, total, loads, walks = _packed_slot_loads(512, views, coverage=False)
    assert total == sum(16 * (sum(v) + 100) + sum(range(32, 513, 32)) for v in views)
    assert sum(loads) >= 0.96 * 64 * max(loads) and min(loads) > 0, (min(loads), max(loads), sum(loads) / 64)
    # Lockstep: slot k of the launch runs on die k % 8, and the eight slots of a die walk the same tokens
    # in the same order (one of them fetches a K/V tile from HBM, the others find it in the die's L2).
    # Only the chunk's own block ends where each tile's causal limit puts it: 32 tokens apart.
    for die in range(8):
        lanes = walks[die::8]
        assert len(lanes) == 8
        for lane in lanes[1:]:
            assert len(lane) == len(lanes[0])
            for (kv, t0, t1), (kv0, u0, u1) in zip(lane, lanes[0]):
                assert (kv, t0) == (kv0, u0) and 0 <= t1 - u1 <= 7 * 32


def test_prefill_tiles_are_cut_by_tokens_on_page_group_boundaries():
    """Two prefill requests of one 32-row tile each, one over 30000 context tokens
    in three segments of odd lengths, one over 700: too few tiles to fill the
    machine, so the planner splits them by tokens.  The long tile must come out
    in many pieces (eight parts of its walk side by side on the slots of a die, each cut where a
    die's share ends) that load the dies alike, the short one in at most three; with pages of 16
    tokens every cut inside a segment lies on a 16-token boundary, with pages of
    4 it need not; every visible pair is covered once either way."""
    for page in (16, 4):
        qo, kvp, kvi, lens, flags, chain, sw = [0], [0], [], [], [], [], []
        n_rows = 0
        for r, segments in enumerate(((11111, 9999, 8890), (700,))):
            rows = list(range(n_rows, n_rows + 8))
            n_rows += 8
            for L in segments:
                kvi += list(range(len(kvi), len(kvi) + -(-L // page)))
                kvp.append(len(kvi)); lens.append(L); flags.append(0); chain.append(r)
                sw += rows; qo.append(len(sw))
            kvi += list(range(len(kvi), len(kvi) + -(-(40 + 8) // page)))
            kvp.append(len(kvi)); lens.append(48); flags.append(1); chain.append(r)
            sw += rows; qo.append(len(sw))
        rc, blob, counts = build_plan(qo, kvp, kvi, lens, flags, chain, sw, n_rows, heads=(16, 4, 256), page=page,
                                      dtype=native.VA_BF16, kernel=native.VA_KERNEL_MFMA)
        assert rc == 0
        check_coverage(blob, qo, kvp, lens, flags, sw, n_rows)
        h, items, links, *_ = decode_plan(blob)
        real = [it for it in items if it[2] > 0]
        pieces = {}
        for it in real:
            ls = links[it[0]: it[0] + it[1]]
            long_one = any(int(l[0]) < kvp[3] for l in ls)  # kv_begin inside the first request's tables
            pieces[long_one] = pieces.get(long_one, 0) + 1
        # (the short tile, 748 tokens in two segments, is worth less than a group's share with its set-ups:
        # it may be cut once or twice, not shredded)
        assert pieces[False] <= 3, "the short tile was cut in many pieces"
        assert pieces[True] >= 20, "the long tile was not cut by its tokens"
        # What a workgroup slot costs: the tokens it walks and ~640 more for every segment it stages.  The
        # eight slots of a die walk a tile's eight parts side by side: the dies must come out alike.
        slots = blob[h[H["OFF_WIDE_SLOTS"]]: h[H["OFF_WIDE_SLOTS"]] + h[H["N_WIDE_SLOTS"]] + 1]
        loads = [int(items[a:b, 4].sum()) + 640 * int(items[a:b, 1].sum()) for a, b in zip(slots, slots[1:])]
        dies = [max(loads[d::8]) for d in range(8) if max(loads[d::8]) > 0]
        assert len(dies) >= 4 and max(dies) <= 1.3 * sum(dies) / len(dies), dies
        inner = [int(l[1]) for it in real for l in links[it[0]: it[0] + it[1]] if l[1] > 0]
        assert inner, "no cut inside a segment"
        if page >= 16:
            assert all(t % 16 == 0 for t in inner)
        else:
            assert any(t % 16 for t in inner)
