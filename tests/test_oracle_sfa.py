"""Pins oracle.sfa: dequantisation against a hand-made IEEE rounding, the attention goldens against float64
attention and against invariants that a dropped term, a wrong index or a transposed operand would break."""
import numpy as np
import pytest
import torch

from oracle import sfa
from oracle.compare import count_violations
from oracle.paged import logical_to_physical


def bf16_rne_from_f64(x):
    """float64 -> nearest bfloat16 (ties to even), by integer arithmetic on the float32 bits of the exactly
    representable inputs used below (products of an int8 and a float32 fit float64 exactly)."""
    f32 = np.float32(x)  # exact for our inputs? not in general: round in float64 instead
    m, e = np.frexp(np.abs(x))  # x = m * 2^e, m in [0.5, 1)
    scaled = np.ldexp(m, 8)  # 8 significant bits: [128, 256)
    r = np.rint(scaled)  # numpy rint = ties to even
    out = np.sign(x) * np.ldexp(r, e - 8)
    return np.where(x == 0, 0.0, out)


def test_dequant_is_one_fp32_product_rounded_once_to_bf16():
    g = torch.Generator().manual_seed(0)
    scales = torch.cat([0.005 + 0.015 * torch.rand(60, generator=g), torch.tensor([1e-8, 1.0, 0.0078125, 3.1e-3])])
    vals = torch.arange(-128, 128, dtype=torch.int8)
    for s in scales.tolist():
        kn = vals.repeat(2).reshape(1, 512)
        sc = torch.full((1, 4), s, dtype=torch.float32)
        got = sfa.dequant_nope(kn, sc).to(torch.float64).numpy().reshape(-1)[:256]
        s32 = np.float64(np.float32(s))
        prod32 = np.float32(vals.numpy().astype(np.float64) * s32)  # fp32 product (float64 product is exact)
        want = bf16_rne_from_f64(prod32.astype(np.float64))
        assert np.array_equal(got, want), s


def test_dequant_uses_one_scale_per_128_columns():
    kn = torch.ones((3, 512), dtype=torch.int8)
    sc = torch.tensor([[1.0, 2.0, 4.0, 8.0]] * 3)
    out = sfa.dequant_nope(kn, sc).float()
    for gidx, v in enumerate([1.0, 2.0, 4.0, 8.0]):
        assert (out[:, 128 * gidx:128 * (gidx + 1)] == v).all()


def test_quantize_round_trip_bound():
    g = torch.Generator().manual_seed(1)
    x = (torch.rand((64, 512), generator=g) * 2 - 1).to(torch.bfloat16)
    q, sc = sfa.quantize_nope(x)
    assert q.dtype == torch.int8 and sc.shape == (64, 4) and int(q.abs().max()) <= 127
    back = sfa.dequant_nope(q, sc).float()
    bound = sc.repeat_interleave(128, dim=1) * 0.5 + back.abs() * 2.0 ** -8 + 1e-7
    assert ((back - x.float()).abs() <= bound).all()


def test_packed_row_layout():
    g = torch.Generator().manual_seed(2)
    kn = torch.randint(-128, 128, (5, 512), generator=g, dtype=torch.int8)
    kr = torch.randn((5, 64), generator=g).to(torch.bfloat16)
    sc = torch.rand((5, 4), generator=g)
    rows = sfa.pack_cache_rows(kn, kr, sc)
    assert rows.shape == (5, 656) and rows.dtype == torch.int8
    raw = rows.numpy().view(np.uint8)
    assert np.array_equal(raw[:, :512], kn.numpy().view(np.uint8))
    assert np.array_equal(raw[:, 512:640].copy().view(np.uint16), kr.view(torch.int16).numpy().view(np.uint16))
    assert np.array_equal(raw[:, 640:656].copy().view(np.float32), sc.numpy())
    kn2, kr2, sc2 = sfa.unpack_cache_rows(rows)
    assert torch.equal(kn2, kn) and torch.equal(kr2, kr) and torch.equal(sc2, sc)


def test_cur_seq_clamp_enumerated():
    for act in range(0, 7):
        for s1 in (1, 2, 3):
            for i in range(s1):
                want = act - s1 + 1 + i
                want = 0 if want < 0 else want
                want = 4 if want > 4 else want
                assert sfa.cur_seq_of(act, s1, i, 4) == want
    assert sfa.cur_seq_of(65536, 2, 0, 2048) == 2048 and sfa.cur_seq_of(15, 2, 0, 2048) == 14


def _args(c):
    return (c["q"], c["kn"], c["kr"], c["kn_scales"], c["topk_indices"], c["block_table"], c["act_seq"],
            c["block_size"], c["softmax_scale"], c["topk"])


@pytest.mark.parametrize("dist", ["uniform", "bench"])
def test_goldens_agree_with_float64_attention(dist):
    c = sfa.make_case(2, 8, 2, [700, 90], topk=256, seed=3, dist=dist,
                      softmax_scale=192 ** -0.5 if dist == "bench" else None)
    ref = sfa.attention_fp64(*_args(c))
    for out in (sfa.attention_no_flash(*_args(c)), sfa.attention_flash(*_args(c), s2_tile=64)):
        assert out.dtype == torch.bfloat16 and out.shape == (2, 2, 8, 512)
        # one bf16 rounding of the result plus the bf16 rounding of P (which weighs more where the softmax is
        # peaked, i.e. on the benchmark distribution); a structural mistake is orders of magnitude away
        atol, rtol = (1e-3, 2.0 ** -7) if dist == "uniform" else (5e-3, 2.0 ** -6)
        assert count_violations(out.double(), ref, atol, rtol) == 0


def test_single_selected_token_returns_its_dequantised_row():
    c = sfa.make_case(1, 4, 1, [500], topk=1, seed=4)
    out = sfa.attention_no_flash(*_args(c))
    row = int(logical_to_physical(c["topk_indices"][0, :1], c["block_table"][0], 128)[0])
    want = sfa.dequant_nope(c["kn"][row:row + 1], c["kn_scales"][row:row + 1])[0]
    assert all(torch.equal(out[0, 0, h], want) for h in range(4))
    assert torch.equal(sfa.attention_flash(*_args(c))[0, 0, 0], want)


def test_zero_query_gives_the_mean_value_row():
    c = sfa.make_case(1, 2, 1, [4096], topk=64, seed=5)  # 1/64 is exact in bf16
    c["q"] = torch.zeros_like(c["q"])
    out = sfa.attention_no_flash(*_args(c)).float()
    rows = logical_to_physical(c["topk_indices"][0, :64], c["block_table"][0], 128)
    v = sfa.dequant_nope(c["kn"][rows], c["kn_scales"][rows]).float()
    want = (v / 64.0).sum(0).to(torch.bfloat16).float()
    assert (out[0, 0, 0] - want).abs().max() <= want.abs().max() * 2.0 ** -7


def test_output_is_a_convex_combination_of_value_rows():
    c = sfa.make_case(1, 4, 1, [3000], topk=128, seed=6, dist="bench", softmax_scale=192 ** -0.5)
    out = sfa.attention_no_flash(*_args(c)).float()
    rows = logical_to_physical(c["topk_indices"][0, :128], c["block_table"][0], 128)
    v = sfa.dequant_nope(c["kn"][rows], c["kn_scales"][rows]).float()
    lo, hi = v.min(0).values, v.max(0).values
    slack = (hi - lo) * 2.0 ** -6 + 1e-6
    assert (out[0, 0] >= lo - slack).all() and (out[0, 0] <= hi + slack).all()


def test_entries_past_cur_seq_and_their_order_do_not_matter():
    c = sfa.make_case(2, 4, 2, [300, 40], topk=256, seed=7)
    base = sfa.attention_no_flash(*_args(c))
    poisoned = dict(c)
    tk = c["topk_indices"].clone()
    for bi, act in enumerate(c["act_seq"]):
        for si in range(2):
            n = sfa.cur_seq_of(act, 2, si, 256)
            tk[bi * 2 + si, n:] = -1  # would raise in the page lookup if it were dereferenced
    poisoned["topk_indices"] = tk
    assert torch.equal(sfa.attention_no_flash(*_args(poisoned)), base)
    shuffled = dict(c)
    tk2 = c["topk_indices"].clone()
    n = sfa.cur_seq_of(300, 2, 1, 256)
    tk2[1, :n] = tk2[1, :n][torch.randperm(n, generator=torch.Generator().manual_seed(8))]
    shuffled["topk_indices"] = tk2
    out2 = sfa.attention_no_flash(*_args(shuffled))
    assert count_violations(out2[0, 1].float(), base[0, 1].float(), 1e-6, 2.0 ** -7) == 0
    assert torch.equal(out2[1], base[1])


def test_causal_rows_of_a_multi_token_query_see_different_lengths():
    c = sfa.make_case(1, 2, 2, [100], topk=256, seed=9)
    out = sfa.attention_no_flash(*_args(c))
    # token 0 sees 99 entries, token 1 sees 100: computing token 0 alone with act 99 must give the same row
    solo = dict(c)
    solo["q"] = c["q"][:, :1]
    solo["topk_indices"] = c["topk_indices"][:1]
    solo["act_seq"], solo["s1"] = [99], 1
    assert torch.equal(sfa.attention_no_flash(*_args(solo))[0, 0], out[0, 0])


def test_no_selected_token_leaves_zeros():
    c = sfa.make_case(1, 2, 2, [1], topk=16, seed=10)  # token 0: cur_seq 0, token 1: cur_seq 1
    for out in (sfa.attention_no_flash(*_args(c)), sfa.attention_flash(*_args(c))):
        assert (out[0, 0] == 0).all() and (out[0, 1] != 0).any()


def test_packed_entry_equals_three_tensor_entry():
    c = sfa.make_case(2, 4, 1, [400, 129], topk=128, seed=11)
    rows = sfa.pack_cache_rows(c["kn"], c["kr"], c["kn_scales"])
    qn = c["q"][..., :512].reshape(-1, 512)
    qr = c["q"][..., 512:].reshape(-1, 64)
    for flash in (False, True):
        out = sfa.attention_packed(qn, qr, rows, c["topk_indices"], c["block_table"], c["act_seq"], 4, 128,
                                   c["softmax_scale"], 128, flash=flash, s2_tile=64)
        want = sfa.attention_flash(*_args(c), s2_tile=64) if flash else sfa.attention_no_flash(*_args(c))
        assert torch.equal(out, want)


def test_naive_token_loop_restatement_matches():
    """The reference's golden walks the selected tokens one at a time (offset = page * bs + idx % bs, copy the
    row); doing exactly that on a small case must reproduce the vectorised oracle bit for bit."""
    for c in (sfa.make_case(1, 3, 2, [150], topk=64, seed=12), sfa.make_case(2, 4, 2, [300, 1], topk=128, seed=13)):
        assert torch.equal(sfa.attention_no_flash_token_loop(*_args(c)), sfa.attention_no_flash(*_args(c)))
