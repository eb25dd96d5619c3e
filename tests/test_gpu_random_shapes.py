"""GPU parity over randomly drawn shapes: every operator against its CPU oracle.

The named tests pin the reference's cases and the edge cases one by one; this one walks a seeded sample of the space
between them (batch, query tokens per sequence, lengths around the tile / page / selection boundaries, page sizes,
selection sizes, head counts, entry points, cache forms), with the same checkers and the same bars.
"""
import random

import pytest
import torch

from oracle import indexer as oi
from oracle import sfa as osfa

from _cases import run_indexer, run_sfa, sfa_golden
from test_gpu_indexer import check_topk
from test_gpu_sfa import check

pytestmark = pytest.mark.gpu

EDGES = [0, 1, 2, 15, 127, 128, 129, 2047, 2048, 2049, 4095, 4096, 4097]


def draw_len(rng, hi):
    c = rng.random()
    if c < 0.15:
        return rng.choice(EDGES)
    if c < 0.5:
        return rng.randint(1, 5000)
    return rng.randint(1, hi)


@pytest.mark.parametrize("seed", [101, 202, 303])
def test_indexer_random_shapes(cuda, seed):
    rng = random.Random(seed)
    for i in range(25):
        b, s1 = rng.randint(1, 4), rng.choice([1, 1, 2, 3, 4])
        act = [draw_len(rng, 40000) for _ in range(b)]
        bs = rng.choice([128, 128, 128, 256, 64, 48, 16])
        k = rng.choice([2048, 2048, 512, 64, 1024])
        dist = rng.choice(["bench", "driver"])
        case = oi.make_case(b, s1, act, seed=1000 * seed + i, block_size=bs, selected_count=k, dist=dist)
        try:
            check_topk(case, run_indexer(case, cuda))
        except AssertionError as e:
            raise AssertionError(f"b={b} s1={s1} act={act} block_size={bs} k={k} dist={dist}: {e}") from e


@pytest.mark.parametrize("seed", [404, 505])
def test_attention_random_shapes(cuda, seed):
    rng = random.Random(seed)
    for i in range(20):
        b, s1 = rng.randint(1, 3), rng.choice([1, 1, 2, 3])
        nq = rng.choice([128, 64, 16, 32, 8, 96])
        topk = rng.choice([2048, 2048, 256, 512, 96])
        act = [draw_len(rng, 20000) for _ in range(b)]
        bs = rng.choice([128, 128, 64, 256])
        quant = rng.random() < 0.8
        packed = quant and rng.random() < 0.4
        entry = rng.choice(["d", "p", "d_950"])
        dist = rng.choice(["uniform", "bench"]) if quant else "uniform"
        name = (f"b={b} s1={s1} nq={nq} topk={topk} act={act} block_size={bs} quant={quant} packed={packed} "
                f"entry={entry} dist={dist}")
        case = osfa.make_case(b, nq, s1, act, topk=topk, block_size=bs, seed=1000 * seed + i, quant=quant, dist=dist)
        check(run_sfa(case, cuda, entry=entry, packed=packed), sfa_golden(case), name)


@pytest.mark.parametrize("seed", [404, 505])
def test_attention_pre_quant_random_shapes(cuda, seed):
    """GLM-4.5 attention_pre_quant: token counts around the 32-token tile, hidden sizes on both sides of the two norm
    kernels and with short last splits of the contraction, head counts that put the projection kernel at one, two and
    four stages per workgroup, token counts on both sides of the switch to the prefill-size projection kernel, every
    rotary width, both input distributions."""
    from oracle import attention_pre_quant as oapq
    from test_gpu_attention_pre_quant import check as check_apq
    from test_gpu_attention_pre_quant import run as run_apq
    rng = random.Random(seed)
    for i in range(12):
        t = rng.choice([1, 2, 7, 8, 31, 32, 33, 63, 64, 65, 127, 128, 129, 257, rng.randint(1, 130), rng.randint(128, 400)])
        h = 256 * rng.choice([1, 2, 3, 7, 20, 24, 25, 28, 33, 64])
        kv = rng.choice([1, 1, 2, 4])
        qh = kv * rng.choice([1, 2, 6, 12])
        half = rng.choice([1, 2, 7, 16, 32, 32, 33, 64])
        case = oapq.make_case(t, h=h, q_heads=qh, kv_heads=kv, half=half, seed=seed + i, realistic=rng.random() < 0.8)
        print(f"attention_pre_quant case {i}: t {t} h {h} heads {qh}+{kv}+{kv} half {half}", flush=True)
        check_apq(case, run_apq(case, cuda))


@pytest.mark.parametrize("seed", [606])
def test_mla_prolog_prefill_random_shapes(cuda, seed):
    """MLA prolog at 128 tokens and more (the kernels that own an output tile): token counts that end inside a 128- or
    256-token tile, contractions of one to several 1024-row splits with a short last one, one to three stages of the
    int8 product, several heads per 128-column output tile."""
    from oracle import mla_prolog as omla
    from test_gpu_mla_prolog import check as check_mla
    from test_gpu_mla_prolog import run as run_mla
    rng = random.Random(seed)
    for i in range(5):
        t = rng.choice([128, 129, 191, 256, 257, rng.randint(128, 330)])
        h = 256 * rng.choice([1, 2, 5, 8, 9])
        r = 128 * rng.choice([1, 2, 3])
        n = rng.choice([2, 4, 6])
        s1 = rng.choice([1, 1, 2])
        b = (t + s1 - 1) // s1
        print(f"mla_prolog case {i}: b {b} s1 {s1} h {h} r {r} n {n}", flush=True)
        case = omla.make_case(b, s1, 300, seed=seed + i, h=h, q_lora_rank=r, n=n)
        check_mla(case, run_mla(case, cuda, entry="mla_prolog_quant_p"))


@pytest.mark.parametrize("seed", [707])
def test_topk_random_shapes(cuda, seed):
    """Standalone top-k: ranks 1 to 4, any axis, rows on both sides of the whole-row sort's limit, k up to the row;
    normal values, heavy ties, quarter-integers, and rows with infinities, signed zeros and magnitudes from 1e-40 to 1e38."""
    from test_gpu_topk import check as check_topk_op
    rng = random.Random(seed)
    g = torch.Generator().manual_seed(seed)
    for i in range(40):
        rank = rng.choice([1, 2, 2, 3, 4])
        n = rng.choice([1, 2, 7, 64, 128, 1000, 4096, 4097, 8192, 8193, 20000, rng.randint(1, 70000)])
        others = [rng.randint(1, 9 if n < 5000 else 3) for _ in range(rank - 1)]
        dim = rng.randint(-rank, rank - 1)
        shape = list(others)
        shape.insert(dim % rank, n)
        k = rng.choice([1, n, min(n, 2048), rng.randint(1, min(n, 4100))])
        if n > 8192:
            k = min(k, 2048)
        largest = rng.random() < 0.6
        kind = rng.choice(["randn", "ties", "ints", "special"])
        x = torch.randn(shape, generator=g)
        if kind == "ties":
            x = torch.randint(-3, 4, shape, generator=g).float()
        elif kind == "ints":
            x = torch.randint(-1000, 1000, shape, generator=g).float() * 0.25
        elif kind == "special":
            x = x * torch.tensor(10.0) ** torch.randint(-40, 38, shape, generator=g).float()
            for v in (float("inf"), float("-inf"), -0.0, 0.0):
                x.view(-1)[torch.randint(0, x.numel(), (max(1, x.numel() // 50),), generator=g)] = v
        print(f"topk case {i}: shape {shape} dim {dim} k {k} largest {largest} {kind}", flush=True)
        check_topk_op(x, k, dim, largest, cuda)


@pytest.mark.parametrize("seed", [808])
def test_paged_gather_random_shapes(cuda, seed):
    """Paged gather: every dtype, row widths that take the 16-, 4-, 2- and 1-byte copy paths, the column-limited
    entry, page sizes from 1, index counts around the 32-row workgroup; bit-exact."""
    from oracle import paged
    from pypto_amd.experimental import gather_in_l1, gather_in_ub
    rng = random.Random(seed)
    g = torch.Generator().manual_seed(seed)
    for i in range(40):
        dtype = rng.choice([torch.int8, torch.float32, torch.bfloat16, torch.float16, torch.int32])
        hidden = rng.choice([1, 3, 7, 8, 16, 36, 64, 129, 512, 576, 656, 1000, rng.randint(1, 1200)])
        size = hidden if rng.random() < 0.6 else rng.randint(1, hidden)
        bs = rng.choice([1, 3, 4, 16, 128])
        nblk = rng.randint(1, 60)
        k = rng.choice([1, 31, 32, 33, 2048, rng.randint(1, 3000)])
        n = nblk * bs
        src = torch.randint(-100, 100, (n, hidden), generator=g).to(dtype)
        page = torch.randperm(nblk, generator=g).to(torch.int32).reshape(1, nblk)
        idx = torch.randint(0, n, (1, k), generator=g, dtype=torch.int32)
        name = f"{dtype} hidden {hidden} size {size} block {bs} pages {nblk} k {k}"
        if size != hidden:
            out = gather_in_l1(src.to(cuda), idx.to(cuda), page.to(cuda), bs, size).cpu()
        else:
            out = gather_in_ub(src.to(cuda), idx.to(cuda), page.to(cuda), bs, -2).cpu()
        want = paged.paged_gather(src, idx[0], page[0], bs)[:, :size]
        assert torch.equal(out.contiguous().view(torch.uint8), want.contiguous().view(torch.uint8)), name


@pytest.mark.parametrize("seed", [909])
def test_select_experts_random_shapes(cuda, seed):
    """Expert selection: 1 to 16 groups of 1 to 32 experts, any number of groups kept, top-k up to 32, token counts around
    the 64-token workgroup, both dtypes of either operand, every flag."""
    from oracle import select_experts as ose
    from test_gpu_select_experts import check as check_se
    rng = random.Random(seed)
    for i in range(40):
        n_group = rng.choice([1, 2, 4, 8, 8, 16])
        per = min(rng.choice([1, 2, 4, 8, 16, 20, 32]), 256 // n_group)
        topk_group = rng.randint(1, n_group)
        top_k = rng.randint(1, min(topk_group * per, 32))
        t = rng.choice([1, 2, 7, 63, 64, 65, 1000, rng.randint(1, 3000)])
        ld, bd = rng.choice([torch.float32, torch.bfloat16]), rng.choice([torch.float32, torch.bfloat16])
        dist = rng.choice(["normal", "uniform"])
        renorm, neg, scale = rng.random() < 0.7, rng.random() < 0.3, rng.choice([1.0, 2.5, 0.5])
        print(f"select_experts case {i}: t {t} experts {n_group}x{per} keep {topk_group} top_k {top_k} {ld} {bd} {dist} "
              f"renorm {renorm} neg {neg} scale {scale}", flush=True)
        logits, bias = ose.make_case(t, n_group * per, seed=1000 * seed + i, logits_dtype=ld, bias_dtype=bd, dist=dist)
        check_se(logits, bias, top_k, renorm, topk_group, n_group, cuda, scale=scale, neg=neg)


@pytest.mark.parametrize("seed", [1010])
def test_gqa_random_shapes(cuda, seed):
    """Paged GQA decode: 1 to 8 KV heads with 1 to 16 query heads each, 1 to 3 query tokens, page sizes 32 to 256,
    lengths around the page and chunk boundaries, both input distributions."""
    from oracle import gqa as og
    from test_gpu_gqa import check as check_gqa
    from test_gpu_gqa import run as run_gqa
    rng = random.Random(seed)
    for i in range(12):
        b, s1 = rng.randint(1, 6), rng.choice([1, 1, 2, 3])
        nkv = rng.choice([1, 1, 2, 4, 8])
        nq = nkv * rng.choice([1, 2, 4, 6, 8, 12, 16])
        act = [max(draw_len(rng, 12000), s1) for _ in range(b)]
        bs = rng.choice([128, 128, 64, 256, 32])
        dist = rng.choice(["normal", "uniform"])
        name = f"b={b} s1={s1} nq={nq} nkv={nkv} act={act} block_size={bs} dist={dist}"
        print(f"gqa case {i}: {name}", flush=True)
        case = og.make_case(b, s1, nq, nkv, act, block_size=bs, seed=1000 * seed + i, dist=dist)
        check_gqa(run_gqa(case, cuda), case, name)


@pytest.mark.parametrize("seed", [1111])
def test_prolog_random_shapes(cuda, seed):
    """Indexer prolog, MLA prolog (int8 and bf16 forms, both entries) and the fused prolog: token counts around the 32- and
    128-token tiles and the switch to the prefill kernels, hidden sizes of one to many 256-row splits, 1 to 3 stages of the
    int8 product, 2 to 16 heads, 32 to 128 index heads; the fused call must also give the bits of the separate calls."""
    from oracle import indexer_prolog as oip
    from oracle import mla_prolog as omla
    from test_gpu_indexer_prolog import check as check_ip
    from test_gpu_indexer_prolog import run as run_ip
    from test_gpu_mla_indexer_prolog import check_against_oracle, run_fused, run_separate, same_as_separate
    from test_gpu_mla_prolog import check as check_mla
    from test_gpu_mla_prolog import check_bf16_form
    from test_gpu_mla_prolog import run as run_mla
    rng = random.Random(seed)
    for i in range(6):
        s1 = rng.choice([1, 1, 2, 3, 4])
        t = rng.choice([1, 2, 31, 32, 33, 64, 100, 127, 128, 129, 200, 257, rng.randint(1, 300)])
        b = max(1, t // s1)
        h = 256 * rng.choice([1, 2, 4, 5, 8])
        r = 128 * rng.choice([1, 2, 3])
        n, n_idx = rng.choice([2, 4, 6, 8, 16]), rng.choice([32, 64, 96, 128])
        print(f"prolog case {i}: b {b} s1 {s1} h {h} r {r} heads {n} index heads {n_idx}", flush=True)
        case = oip.make_case(b, s1, 600, seed=1000 * seed + i, h=h, q_lora_rank=r, n=n_idx, hadamard=rng.choice(["uniform", "walsh"]))
        check_ip(case, run_ip(case, cuda))
        qb = rng.random() < 0.7
        rr = r if qb else 256 * rng.choice([1, 2])
        entry = "mla_prolog_quant_p" if (b * s1 >= 128 or rng.random() < 0.3) else "mla_prolog_quant_d"
        case = omla.make_case(b, s1, 300, seed=1000 * seed + i, h=h, q_lora_rank=rr, n=n, quant_b=qb)
        got = run_mla(case, cuda, entry=entry)
        check_mla(case, got) if qb else check_bf16_form(case, got, outliers=1e-4)
        mla_case, idx_case = omla.make_fused_case(b, s1, 600, seed=1000 * seed + i, n_idx=n_idx, h=h, q_lora_rank=r, n=n)
        fused = run_fused(mla_case, idx_case, cuda, entry="mla_indexer_prolog_quant_p" if b * s1 >= 128 else "mla_indexer_prolog_quant_d")
        check_against_oracle(mla_case, idx_case, fused)
        same_as_separate(fused, run_separate(mla_case, idx_case, cuda), idx_case)
