"""Pins oracle.indexer: integer dot products by brute force, both fp16 roundings by hand, the score formula by an
independent per-element loop, and the selection rules on hand-made rows."""
import numpy as np
import pytest
import torch

from oracle import indexer as oi
from oracle.paged import paged_gather


def f16_rne(x64):
    """float64 -> nearest fp16 value (ties to even) by integer arithmetic: 11 significant bits in the normal
    range, multiples of 2^-24 below 2^-14 (subnormals)."""
    x64 = np.asarray(x64, dtype=np.float64)
    m, e = np.frexp(np.abs(x64))
    normal = np.sign(x64) * np.ldexp(np.rint(np.ldexp(m, 11)), e - 11)
    sub = np.sign(x64) * np.ldexp(np.rint(np.ldexp(np.abs(x64), 24)), -24)
    return np.where(x64 == 0, 0.0, np.where(np.abs(x64) < 2.0 ** -14, sub, normal))


def test_relu_scale_fp16_rounding_by_hand():
    # every integer dot product the kernel can see is below 2^21; relu(x) / 2048 rounded to fp16
    xs = np.concatenate([np.arange(0, 5000), np.array([2047, 2048, 2049, 4095, 4097, 65535, 65537, 2064512]),
                         np.random.default_rng(0).integers(0, 2064513, 20000)]).astype(np.int64)
    t = (torch.from_numpy(xs).to(torch.int32).float().relu() * oi.SCORE_SHIFT).to(torch.float16).double().numpy()
    assert np.array_equal(t, f16_rne(xs / 2048.0))
    neg = torch.tensor([-1, -2048, -2064512], dtype=torch.int32)
    assert ((neg.float().relu() * oi.SCORE_SHIFT).to(torch.float16) == 0).all()


def test_w_scale_is_one_fp16_product():
    g = torch.Generator().manual_seed(1)
    qs = (0.005 + 0.015 * torch.rand((7, 64), generator=g)).to(torch.float16)
    w = (torch.randn((7, 64), generator=g) / 8).to(torch.float16)
    got = oi.w_scale_of(qs, w).double().numpy()
    want = f16_rne(qs.double().numpy() * w.double().numpy())  # product of two fp16 is exact in float64
    assert (np.abs(want) < 2.0 ** -14).any()  # the case covers fp16 subnormals
    assert np.array_equal(got, want)


def test_scores_match_an_independent_per_element_loop():
    c = oi.make_case(2, 2, [37, 300], seed=2)
    sc = oi.scores(c["query"], c["q_scale"], c["key_cache"], c["k_scale"], c["weights"], c["act_seq"],
                   c["block_table"], 2)
    ex = oi.scores_exact(c["query"], c["q_scale"], c["key_cache"], c["k_scale"], c["weights"], c["act_seq"],
                         c["block_table"], 2)
    q = c["query"].numpy().astype(np.int64)
    keys = c["key_cache"].reshape(-1, 128).numpy().astype(np.int64)
    ks = c["k_scale"].reshape(-1).double().numpy()
    qs, w = c["q_scale"].double().numpy(), c["weights"].double().numpy()
    rng = np.random.default_rng(3)
    for _ in range(40):
        b = int(rng.integers(0, 2)); s = int(rng.integers(0, 2)); n = int(rng.integers(0, c["act_seq"][b]))
        row = int(c["block_table"][b, n // 128]) * 128 + n % 128
        tot = 0.0
        for h in range(64):
            dot = int((q[b * 2 + s, h] * keys[row]).sum())  # exact integer arithmetic
            y = float(f16_rne(max(dot, 0) / 2048.0))
            tot += float(f16_rne(qs[b * 2 + s, h] * w[b * 2 + s, h])) * y
        want = tot * ks[row]
        assert abs(float(ex[b * 2 + s, n]) - want) <= 1e-12 * max(1.0, abs(want))
        assert abs(float(sc[b * 2 + s, n]) - want) <= 1e-5 * float(ex[b * 2 + s].abs().max())
    assert (sc[:, 37:128][0:2] == 0).all()  # beyond the sequence nothing is written


def test_selection_rules():
    scores = torch.tensor([[0.5, 2.0, -1.0, 2.0, 0.25, 9.0, 9.0, 9.0],
                           [0.5, 2.0, -1.0, 2.0, 0.25, 9.0, 9.0, 9.0]])
    # one sequence of length 6, two query tokens: eff_seq = 5 and 6
    out = oi.select(scores, [6], 2, 4)
    assert out.shape == (2, 1, 4)
    assert out[0, 0].tolist() == [1, 3, 0, 4]  # ties by ascending index, columns >= 5 invisible
    assert out[1, 0].tolist() == [5, 1, 3, 0]
    short = oi.select(scores[:1], [3], 1, 4)
    assert short[0, 0].tolist() == [1, 0, 2, -1]  # fewer valid tokens than slots: -1 fills
    assert oi.select(scores[:1], [0], 1, 4)[0, 0].tolist() == [-1] * 4
    assert oi.eff_seq_of(10, 4, 0) == 7 and oi.eff_seq_of(10, 4, 3) == 10


def test_paged_scatter_round_trip():
    c = oi.make_case(3, 1, [130, 5, 256], seed=4, dist="driver")
    # key n of sequence b sits where the page table says
    g = torch.Generator().manual_seed(4)
    keys2d = c["key_cache"].reshape(-1, 128)
    for b, L in enumerate(c["act_seq"]):
        got = paged_gather(keys2d, torch.arange(L), c["block_table"][b], 128)
        assert got.shape == (L, 128)
    k_log = torch.arange(2 * 200 * 4, dtype=torch.int32).reshape(2, 200, 4)
    table = torch.tensor([[3, 0], [1, 2]], dtype=torch.int32)
    cache = oi.scatter_to_cache(k_log, table, 4, 128)
    for b in range(2):
        assert torch.equal(paged_gather(cache.reshape(-1, 4), torch.arange(200), table[b], 128), k_log[b])


def test_driver_style_case_respects_quantisation_ranges():
    c = oi.make_case(2, 2, [300, 64], seed=5, dist="driver")
    assert int(c["query"].abs().max()) <= 127 and int(c["key_cache"].abs().max()) <= 127
    assert float(c["q_scale"].min()) >= 1e-3 - 1e-6 and c["q_scale"].dtype == torch.float16
    out = oi.lightning_indexer(c["query"], c["q_scale"], c["key_cache"], c["k_scale"], c["weights"], c["act_seq"],
                               c["block_table"], 2, 2048)
    assert out.shape == (4, 1, 2048) and (out[0, 0, 299:] == -1).all() and (out[1, 0, 300:] == -1).all()
    assert sorted(out[1, 0, :300].tolist()) == list(range(300))


def test_fp32_scale_variant():
    """The fp32-scale variant (scales kept in fp32; not in the reference, whose operator takes fp16): with fp32 tensors
    that hold fp16 values it gives the bits of the fp16 form (every product it forms is then the same number); with
    general fp32 scales w_scale is the fp32 product rounded to fp16 by hand, and the score follows the formula in
    float64 to fp32 accuracy."""
    case = oi.make_case(2, 2, [300, 77], seed=9)
    args = lambda c: (c["query"], c["q_scale"], c["key_cache"], c["k_scale"], c["weights"], c["act_seq"], c["block_table"], c["s1"])  # noqa: E731
    as32 = dict(case, q_scale=case["q_scale"].float(), k_scale=case["k_scale"].float())
    assert torch.equal(oi.scores(*args(as32)), oi.scores(*args(case)))
    c32 = oi.make_case(2, 2, [300, 77], seed=9, scale_dtype=torch.float32)
    assert c32["q_scale"].dtype == torch.float32 and not torch.equal(c32["q_scale"], c32["q_scale"].half().float())
    ws = oi.w_scale_of(c32["q_scale"], c32["weights"])
    prod32 = (c32["q_scale"].double() * c32["weights"].double()).float()   # the fp32 product (one rounding of the exact one)
    assert torch.equal(ws.double(), torch.from_numpy(f16_rne(prod32.double().numpy())))
    # the formula end to end in float64 from the same w_scale, page by page through the table
    sc = oi.scores(*args(c32))
    t, nh, d = c32["query"].shape
    for r in range(t):
        bi = r // 2
        for tok in (0, 1, min(130, c32["act_seq"][bi] - 1), c32["act_seq"][bi] - 1):
            page, off = int(c32["block_table"][bi, tok // 128]), tok % 128
            dot = (c32["query"][r].long() @ c32["key_cache"][page, off, 0].long()).clamp(min=0)
            y = torch.from_numpy(f16_rne((dot.double() / 2048).numpy()))
            want = float((ws[r].double() * y).sum() * c32["k_scale"][page, off, 0].double())
            assert abs(float(sc[r, tok]) - want) <= 1e-5 * max(abs(want), 1e-6)
