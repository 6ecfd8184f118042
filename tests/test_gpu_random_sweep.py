"""Seeded random sweeps of decode and batched prefill against the CPU oracle:
page sizes 1..64, every supported head layout and head_dim, bf16/f16, full and
partial rotation, 3-D mRoPE with compressed spans, 0..3 shared or context
blocks of 0..2500 tokens, both kernels.  The fixed scenarios of the other
files follow the reference's tests; these cover the combinations between them.
Every case prints its parameters before it runs."""

import random

import pytest
import torch

from async_llm_amd.shared_cache import CacheBlock, PrefillSpec, WorkerGroup
from tests.test_gpu_decode import Pages
from tests.util import make_op_and_pool, run_decode_parity, run_prefill_parity

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda")


def mrope_sections(rotary):
    half = rotary // 2
    return half // 2, half // 4, half - half // 2 - half // 4


@pytest.mark.parametrize("seed", [11, 12])
def test_random_prefill_batches(seed):
    rng = random.Random(seed)
    for case in range(40):
        page = rng.choice([1, 4, 16, 16, 16, 32, 64])
        heads = rng.choice([(4, 4, 64), (8, 2, 64), (8, 2, 128), (16, 2, 128), (8, 2, 256), (16, 4, 256), (16, 1, 256),
                            (4, 4, 256)])
        dtype = rng.choice([torch.bfloat16, torch.bfloat16, torch.float16])
        D = heads[2]
        mrope = rng.random() < 0.25
        rotary = D // 2 if mrope else rng.choice([D, D // 2])
        lens = [rng.choice([5, 16, 33, 96, 130, 257, 400, 777]) for _ in range(rng.randint(0, 3))]
        reqs = [(rng.choice([1, 7, 32, 33, 64, 100, 150]), rng.choice([0, 3, 16, 40, 200, 333]))
                for _ in range(rng.randint(1, 3))]
        print(f"prefill seed {seed} case {case}: page {page} heads {heads} {dtype} rotary {rotary} mrope {mrope} "
              f"blocks {lens} requests {reqs}", flush=True)
        total_pages = sum(-(-n // page) for n in lens) + sum(-(-(p + n) // page) for n, p in reqs) + 4
        op, cpu_pool, dev_pool, gen = make_op_and_pool(
            DEV, dtype, heads, page, total_pages, 1e4, rotary_dim=rotary,
            mrope_section=mrope_sections(rotary) if mrope else None, seed=1000 * seed + case, scale=0.5, max_pos=4096)
        blocks, first = [], 0
        for length in lens:
            b = CacheBlock(DEV, page)
            n_pages = -(-length // page)
            b.grow_pages(torch.arange(first, first + n_pages) * page, length)
            if mrope:
                b.mrope_span_override = length // 2 + 1
            blocks.append(b)
            first += n_pages
        specs = []
        for w, (n, prefix) in enumerate(reqs):
            n_pages = -(-(prefix + n) // page)
            pages = torch.arange(first, first + n_pages, dtype=torch.int32) * page
            first += n_pages
            rel = None
            if mrope and w % 2 == 0:
                p = torch.arange(n)
                rel = torch.stack([p // 8, p // 4, p % 4])
            context = blocks[rng.randint(0, len(blocks)):] if blocks else []
            specs.append(PrefillSpec(context, pages, n, prefix, prefix // 2 if mrope else prefix, rel))
        run_prefill_parity(op, cpu_pool, dev_pool, specs, 1e4, gen, scale=0.5)


def test_random_prefill_batches_with_large_scores():
    """Keys and queries of standard deviation 2 per element: scores of standard deviation 4 (natural units) that
    reach +-20 over contexts of a few thousand tokens, so the softmax is close to one-hot and a query rounded
    anywhere else than where the reference rounds it (say, after a multiplication by the softmax scale) moves
    the output by far more than the tolerance.  Longer context blocks than the sweeps above: the interior of
    the wide kernel's walk (its steady loop) does most of the work here."""
    rng = random.Random(31)
    for case in range(24):
        page = rng.choice([1, 4, 16, 16, 16, 32, 64])
        heads = rng.choice([(4, 4, 64), (8, 2, 64), (8, 2, 128), (16, 2, 128), (8, 2, 256), (16, 4, 256), (16, 1, 256),
                            (32, 8, 128)])
        dtype = rng.choice([torch.bfloat16, torch.bfloat16, torch.float16])
        D = heads[2]
        rotary = rng.choice([D, D // 2])
        lens = [rng.choice([5, 33, 257, 400, 777, 1200, 2049, 3100]) for _ in range(rng.randint(1, 4))]
        reqs = [(rng.choice([1, 33, 64, 100, 150, 260, 500]), rng.choice([0, 3, 16, 200, 333, 1000]))
                for _ in range(rng.randint(1, 3))]
        print(f"large-score prefill case {case}: page {page} heads {heads} {dtype} rotary {rotary} blocks {lens} "
              f"requests {reqs}", flush=True)
        total_pages = sum(-(-n // page) for n in lens) + sum(-(-(p + n) // page) for n, p in reqs) + 4
        op, cpu_pool, dev_pool, gen = make_op_and_pool(DEV, dtype, heads, page, total_pages, 1e4, rotary_dim=rotary,
                                                       seed=31000 + case, scale=2.0, max_pos=8192)
        blocks, first = [], 0
        for length in lens:
            b = CacheBlock(DEV, page)
            n_pages = -(-length // page)
            b.grow_pages(torch.arange(first, first + n_pages) * page, length)
            blocks.append(b)
            first += n_pages
        specs = []
        for n, prefix in reqs:
            n_pages = -(-(prefix + n) // page)
            pages = torch.arange(first, first + n_pages, dtype=torch.int32) * page
            first += n_pages
            specs.append(PrefillSpec(blocks[rng.randint(0, len(blocks) - 1):], pages, n, prefix))
        run_prefill_parity(op, cpu_pool, dev_pool, specs, 1e4, gen, scale=2.0)


@pytest.mark.parametrize("seed", [21, 22])
def test_random_decode_views(seed):
    rng = random.Random(seed)
    for case in range(40):
        page = rng.choice([1, 4, 16, 16, 16, 32])
        heads = rng.choice([(4, 4, 64), (8, 2, 64), (8, 8, 128), (32, 2, 128), (16, 4, 256), (16, 2, 256), (16, 1, 256),
                            (4, 4, 256)])
        D = heads[2]
        dtype = rng.choice([torch.bfloat16, torch.bfloat16, torch.float16])
        mrope = rng.random() < 0.25
        rotary = D // 2 if mrope else rng.choice([D, D // 2, D // 4])
        shared_lens = [rng.choice([0, 3, 64, 700, 1500, 2500]) for _ in range(rng.randint(0, 2))]
        lens = [[rng.choice([0, 1, 2, 15, 16, 17, 100, 255, 640, 1000, 1800]) for _ in range(rng.randint(1, 3))]
                for _ in range(rng.randint(1, 9))]
        kernel = rng.choice(["auto", "auto", "generic"])
        print(f"decode seed {seed} case {case}: page {page} heads {heads} {dtype} rotary {rotary} mrope {mrope} "
              f"kernel {kernel} shared {shared_lens} private {lens}", flush=True)
        total = (sum(-(-n // page) + 1 for n in shared_lens) + sum(-(-n // page) + 2 for ls in lens for n in ls)
                 + len(lens) + 8)
        op, cpu_pool, dev_pool, gen = make_op_and_pool(
            DEV, dtype, heads, page, total, 1e6, rotary_dim=rotary,
            mrope_section=mrope_sections(rotary) if mrope else None, seed=1000 * seed + case, scale=0.7,
            kernel=kernel, max_pos=16384)
        pages = Pages(page)
        span = (lambda n: n // 2 + 1) if mrope else (lambda n: None)
        shared = [pages.block(n, span=span(n)) for n in shared_lens]
        views, targets = [], []
        for ls in lens:
            mine = [pages.block(n, span=span(n)) for n in ls]
            views.append(shared[rng.randint(0, len(shared)):] + mine)
            targets.append(mine[-1])
        run_decode_parity(op, cpu_pool, dev_pool, WorkerGroup(cache_structure=views, write_to=targets), pages, 1e6, gen,
                          scale=0.7)
