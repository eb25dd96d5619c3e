"""GPU parity over randomly drawn shapes: lightning indexer and sparse flash attention against the CPU oracle.

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
