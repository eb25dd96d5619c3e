"""GPU parity: MLA prolog, int8 form (HIP, through the C ABI) against the CPU oracle.

Bar.  The reference compares (deepseekv32_mla_prolog_quant.py:679-697): q_nope and q_rope with rtol 0.0078125 /
atol 0.005, the int8 tensors (q_norm, kv_cache) with an absolute tolerance of 1, the fp32 scales with rtol 0.005 /
atol 2.5e-5 and the rope cache with rtol 0.0078125 / atol 1e-4.  Every stage here reproduces the operator's rounding
points; what differs from the oracle is the summation order of the fp32 matmuls and of the RmsNorm sums, which now and
then moves a value across a bf16 rounding boundary.  So, against the oracle evaluated with the operator's epsilons:
int8 values within 1 everywhere and equal in at least 98 % of the places; scales within two bf16 steps (2^-6
relative: a scale follows the largest value of its row, which is a bf16 rounding of the product carried through the
norm's own bf16 rounding - either can fall the other way) and bit-equal in most rows.  A flipped q_norm value moves the 24576 products of its token by up to one int8 step of
that token, which takes a few of that token's q_nope values out of the tight tolerance - the reference's comparator
allows 0.5 % of such outliers (utils/compare.py:16, max_error_ratio); here the same 0.5 %, none beyond 3 x the
tolerance, and none at all on a token whose q_norm row and scale are the golden's (with a short q_lora_rank one int8
step is a larger share of a product, and 0.2 % of the elements were seen outside).  The downstream stages are also checked on their own: from the product's own q_norm /
q_norm_scale the oracle's q_nope and q_rope must be met with no outlier at all.

The rope cache (check_rope_cache): a rope key is a cos + b sin of two bf16 roundings of x @ w_kr.  A rounding that fell
the other way moves a (or b) by one bf16 step and the key by that step times |cos| (|sin|); when the two terms cancel
that is more than 2^-7 of the result.  So: every key within the reference's tolerance plus that move (computed from
the oracle's own a and b), and at most 0.1 % of them outside the plain tolerance.
"""
import pytest
import torch

from oracle import mla_prolog as op

pytestmark = pytest.mark.gpu
EPS = 1e-5


SMALL = 1 << 16
FEW = 3  # a fraction bar on a small sample allows at least this many values (one flipped rounding shows in two or three)


def bf16_step(v):
    """Distance between neighbouring bf16 values at |v| (8 significant bits)."""
    return torch.exp2(torch.floor(torch.log2(v.float().abs().clamp(min=2.0 ** -126))) - 7)


def check_rope_cache(case, got_cache, gold_cache, eps=EPS, min_equal=0.95):
    rows = case["cache_index"]   # (one cache row per token: make_case draws distinct positions)
    a, b = got_cache.view(-1, 64)[rows].float(), gold_cache.view(-1, 64)[rows].float()
    assert torch.isfinite(a).all(), "kr_cache"
    t = a.shape[0]
    pre = op.intermediates(case, eps, eps)["kv"][:, 512:].float()   # the bf16 products, before the rotary embedding
    pre = pre.reshape(t, 32, 2).permute(0, 2, 1).reshape(t, 64)      # pairs (2i, 2i+1) -> positions (i, 32+i)
    move = bf16_step(pre) * case["cos"].float().abs() + bf16_step(op.rotate_half(pre)) * case["sin"].float().abs()
    tol = 1e-4 + 0.0078125 * b.abs()
    err = (a - b).abs()
    worst = float((err / (tol + move)).max())
    assert worst <= 1, f"kr_cache: {worst} x the tolerance plus one flipped rounding of x @ w_kr"
    assert int((err > tol).sum()) <= max(1e-3 * err.numel(), FEW), f"kr_cache: {int((err > tol).sum())} of {err.numel()} values outside the plain tolerance"
    assert (a == b).float().mean() >= min_equal, f"kr_cache: only {(a == b).float().mean():.3f} bit-equal"


def run(case, dev, entry="mla_prolog_quant_d", eps=EPS):
    from pypto_amd.deepseek_v32_exp import mla_prolog_quant_impl as impl
    t = case["x"].shape[0]
    n = case["w_uk"].shape[0]
    r = case["w_dq"].shape[1]
    d = {k: v.to(dev) for k, v in case.items()}
    kv, kr, ks = d["kv_cache"].clone(), d["kr_cache"].clone(), d["k_scale_cache"].clone()
    q_norm = torch.zeros((t, r), dtype=d["kv_cache"].dtype, device=dev)   # int8 form: int8; bf16 form: bf16
    q_norm_scale = torch.zeros((t, 1), dtype=torch.float32, device=dev)
    q_nope = torch.zeros((t, n, 512), dtype=torch.bfloat16, device=dev)
    q_rope = torch.zeros((t, n, 64), dtype=torch.bfloat16, device=dev)
    rope_cfg = impl.RopeTileShapeConfig(two_dim=[32, 64], three_dim=[32, 32, 128], four_dim=[16, 128, 128, 128])
    getattr(impl, entry)(d["x"], d["w_dq"], d["w_uq_qr"], d["w_qb_scale"], d["w_uk"], d["w_dkv_kr"], d["gamma_cq"],
                         d["gamma_ckv"], d["cos"], d["sin"], d["cache_index"], kv, kr, ks, q_norm, q_norm_scale, q_nope,
                         q_rope, kv, kr, ks, eps, eps, "PA_BSND", impl.MlaTileConfig(), rope_cfg)
    torch.cuda.synchronize()
    return {"q_norm": q_norm.cpu(), "q_norm_scale": q_norm_scale.cpu(), "q_nope": q_nope.cpu(), "q_rope": q_rope.cpu(),
            "kv_cache": kv.cpu(), "kr_cache": kr.cpu(), "k_scale_cache": ks.cpu()}


def check(case, got, eps=EPS):
    gold = op.mla_prolog(case, eps, eps)
    rows = case["cache_index"]

    def ints(a, b, name):
        diff = (a.int() - b.int()).abs()
        assert diff.max() <= 1, f"{name}: off by {int(diff.max())}"
        assert (diff == 0).float().mean() >= 0.98, f"{name}: {(diff != 0).float().mean():.4f} of the values differ"

    def scales(a, b, name, min_equal):
        a, b = a.float().flatten(), b.float().flatten()
        assert torch.isfinite(a).all(), name
        assert ((a - b).abs() <= 2.0 ** -6 * b.abs() + 1e-8).all(), f"{name}: {float(((a - b).abs() / b.abs()).max())}"
        assert (a == b).float().mean() >= min_equal, f"{name}: only {(a == b).float().mean():.3f} bit-equal"

    def floats(a, b, name, rtol, atol, min_equal, outliers=0.0):
        a, b = a.float(), b.float()
        assert torch.isfinite(a).all(), name
        ratio = (a - b).abs() / (atol + rtol * b.abs())
        assert int((ratio > 1).sum()) <= (max(outliers * ratio.numel(), FEW) if outliers else 0) and ratio.max() <= 3, \
            f"{name}: {int((ratio > 1).sum())} values outside rtol {rtol} atol {atol}, worst {float(ratio.max())} x"
        # (bit-equality with the golden is asked of samples large enough that one token's flipped q_norm value, which
        # moves a good part of that token's products by a rounding, is not a visible fraction of them)
        if a.numel() >= SMALL or "from the product" in name:
            assert (a == b).float().mean() >= min_equal, f"{name}: only {(a == b).float().mean():.3f} bit-equal"

    ints(got["q_norm"], gold["q_norm"], "q_norm")
    scales(got["q_norm_scale"], gold["q_norm_scale"], "q_norm_scale", 0.80)
    floats(got["q_nope"], gold["q_nope"], "q_nope", 0.0078125, 0.005, 0.85, outliers=5e-3)
    floats(got["q_rope"], gold["q_rope"], "q_rope", 0.0078125, 0.005, 0.85, outliers=5e-3)
    # where those outliers come from: every token that has one carries a q_norm row or scale that differs from the
    # golden's; a token whose quantised row is the golden's has none
    same_q = (got["q_norm"] == gold["q_norm"]).all(1) & (got["q_norm_scale"] == gold["q_norm_scale"]).all(1)
    for name in ("q_nope", "q_rope"):
        a, b = got[name].float(), gold[name].float()
        off = ((a - b).abs() > 0.005 + 0.0078125 * b.abs()).flatten(1).any(1)
        assert not (off & same_q).any(), f"{name}: an outlier on a token whose q_norm row equals the golden's"
    tail_nope, tail_rope = op.query_tail(case, got["q_norm"], got["q_norm_scale"])
    floats(got["q_nope"], tail_nope, "q_nope from the product's q_norm", 0.0078125, 0.005, 0.99)
    floats(got["q_rope"], tail_rope, "q_rope from the product's q_norm", 0.0078125, 0.005, 0.99)
    ints(got["kv_cache"].view(-1, 512)[rows], gold["kv_cache"].view(-1, 512)[rows], "kv_cache")
    scales(got["k_scale_cache"].view(-1, 4)[rows], gold["k_scale_cache"].view(-1, 4)[rows], "k_scale_cache", 0.80)
    check_rope_cache(case, got["kr_cache"], gold["kr_cache"], eps)
    # nothing but the indexed rows of the caches may change
    keep = torch.ones(case["kv_cache"].shape[0] * case["kv_cache"].shape[1], dtype=torch.bool)
    keep[rows] = False
    assert torch.equal(got["kv_cache"].view(-1, 512)[keep], case["kv_cache"].view(-1, 512)[keep])
    assert torch.equal(got["kr_cache"].view(-1, 64)[keep], case["kr_cache"].view(-1, 64)[keep])
    assert torch.equal(got["k_scale_cache"].view(-1, 4)[keep], case["k_scale_cache"].view(-1, 4)[keep])
    # also inside the reference's tolerances of the golden proper (no epsilon)
    g0 = op.mla_prolog(case)
    assert (got["q_norm"].int() - g0["q_norm"].int()).abs().max() <= 1
    assert (got["kv_cache"].view(-1, 512)[rows].int() - g0["kv_cache"].view(-1, 512)[rows].int()).abs().max() <= 1
    bad = (got["q_nope"].float() - g0["q_nope"].float()).abs() > 0.005 + 0.0078125 * g0["q_nope"].float().abs()
    assert bad.float().mean() <= 0.005


def test_reference_case_b4_s2(cuda):
    # the reference's enabled test test_b4_s64k2_pa_nd_bf16_quantb_d: b=4, two new tokens per sequence, model sizes
    case = op.make_case(4, 2, 1024, seed=5)
    check(case, run(case, cuda))


def test_small_sizes_and_ragged_token_tiles(cuda):
    for b, s1, seed in ((1, 1, 11), (37, 1, 12), (9, 4, 13)):
        case = op.make_case(b, s1, 300, seed=seed, h=512, q_lora_rank=256, n=4)
        check(case, run(case, cuda))
    case = op.make_case(3, 2, 300, seed=14, h=1024, q_lora_rank=384, n=6)
    check(case, run(case, cuda, entry="mla_prolog_quant_p"))


def test_decode_batch_model_sizes(cuda):
    case = op.make_case(32, 1, 512, seed=15)
    check(case, run(case, cuda))


def test_reference_prefill_case_t128(cuda):
    # the reference's (skipped, "large shape") prefill test test_b128_s4k4_pa_nd_bf16_quantb_p: 128 tokens, model sizes
    case = op.make_case(128, 1, 1024, seed=17)
    check(case, run(case, cuda, entry="mla_prolog_quant_p"))


def test_prefill_sizes_ragged_token_tiles(cuda):
    # 128 tokens and more run the kernels that own an output tile (256 / 128 tokens per workgroup): token counts that
    # end inside a tile, a contraction that is not a whole number of 1024-row splits, several heads per output tile
    for b, s1, seed, kw in ((130, 1, 31, dict(h=512, q_lora_rank=256, n=4)), (100, 3, 32, dict(h=1280, q_lora_rank=384, n=6)),
                            (257, 2, 33, dict(h=512, q_lora_rank=128, n=2))):
        case = op.make_case(b, s1, 64 * s1 * 2 + 300, seed=seed, **kw)
        check(case, run(case, cuda, entry="mla_prolog_quant_p"))
    case = op.make_case(150, 1, 600, seed=34, h=1280, q_lora_rank=1280, n=6, quant_b=False)
    check_bf16_form(case, run(case, cuda, entry="mla_prolog_quant_p"), outliers=1e-4)


def check_bf16_form(case, got, eps=EPS, outliers=0.0):
    """bf16 form (the reference's tolerances, :686-694: q_norm, kv, kr rtol 2^-7 / atol 1e-4; q_nope, q_rope rtol 2^-7 /
    atol 5e-3): everything within those, and bit-equal in at least 98 % of the places - the difference is the summation
    order of x @ w, which now and then moves a bf16 rounding.  The two RmsNorm outputs (q_norm, the kv cache) may leave
    the tolerance by what one such move does to them: a product element that rounded the other way is one bf16 step
    off, and its normalised value follows by that step times |gamma| / rms (computed per element from the oracle's own
    products), on top of the output's own rounding, which the tolerance covers; at most 0.1 % of the values may need
    it.  `outliers`: the fraction of q_nope / q_rope values that may sit up to 2 x outside (a flipped q_norm value
    moves every product of its token a little; the reference's comparator lets 0.5 % of the values be anywhere)."""
    gold = op.mla_prolog(case, eps, eps)
    rows = case["cache_index"]
    mid = op.intermediates(case, eps, eps)

    def norm_move(pre, gamma, e):
        pre = pre.float()
        inv_rms = 1.0 / torch.sqrt((pre * pre).mean(dim=-1, keepdim=True) + e)
        return bf16_step(pre) * gamma.float().abs().reshape(1, -1) * inv_rms

    def floats(a, b, name, rtol, atol, min_equal=0.98, move=None):
        a, b = a.float(), b.float()
        assert torch.isfinite(a).all(), name
        tol = atol + rtol * b.abs()
        err = (a - b).abs()
        if move is None:
            ratio = err / tol
            assert int((ratio > 1).sum()) <= (max(outliers * ratio.numel(), FEW) if outliers else 0) and ratio.max() <= (2 if outliers else 1), \
                f"{name}: worst {float(ratio.max())} x the tolerance, {int((ratio > 1).sum())} values outside"
        else:
            worst = float((err / (tol + move)).max())
            assert worst <= 1, f"{name}: {worst} x the tolerance plus one flipped rounding of the product"
            assert int((err > tol).sum()) <= max(1e-3 * err.numel(), FEW), f"{name}: {int((err > tol).sum())} of {err.numel()} values outside the plain tolerance"
        if a.numel() >= SMALL or "from the product" in name:
            assert (a == b).float().mean() >= min_equal, f"{name}: only {(a == b).float().mean():.3f} bit-equal"

    floats(got["q_norm"], gold["q_norm"], "q_norm", 0.0078125, 1e-4, move=norm_move(mid["q_a"], case["gamma_cq"], eps))
    floats(got["q_nope"], gold["q_nope"], "q_nope", 0.0078125, 0.005, 0.90)
    floats(got["q_rope"], gold["q_rope"], "q_rope", 0.0078125, 0.005, 0.90)
    if outliers:
        # where the licensed outliers come from: every token that has one carries a q_norm row that differs from the
        # golden's (a rounding of q_a that fell the other way in the kernel's summation order); a token whose q_norm row
        # is the golden's has none - and restarted from the product's own q_norm there is no outlier at all (next check)
        for name, rtol, atol in (("q_nope", 0.0078125, 0.005), ("q_rope", 0.0078125, 0.005)):
            a, b = got[name].float(), gold[name].float()
            off = ((a - b).abs() > atol + rtol * b.abs()).flatten(1).any(1)
            same_q_norm = (got["q_norm"] == gold["q_norm"]).all(1)
            assert not (off & same_q_norm).any(), f"{name}: an outlier on a token whose q_norm row equals the golden's"
    tail_nope, tail_rope = op.query_tail(case, got["q_norm"], None)
    floats(got["q_nope"], tail_nope, "q_nope from the product's q_norm", 0.0078125, 0.005, 0.99)
    floats(got["q_rope"], tail_rope, "q_rope from the product's q_norm", 0.0078125, 0.005, 0.99)
    floats(got["kv_cache"].view(-1, 512)[rows], gold["kv_cache"].view(-1, 512)[rows], "kv_cache", 0.0078125, 1e-4,
           move=norm_move(mid["kv"][:, :512], case["gamma_ckv"], eps))
    check_rope_cache(case, got["kr_cache"], gold["kr_cache"], eps)
    keep = torch.ones(case["kv_cache"].shape[0] * case["kv_cache"].shape[1], dtype=torch.bool)
    keep[rows] = False
    assert torch.equal(got["kv_cache"].view(-1, 512)[keep], case["kv_cache"].view(-1, 512)[keep])
    assert torch.equal(got["kr_cache"].view(-1, 64)[keep], case["kr_cache"].view(-1, 64)[keep])
    assert torch.equal(got["k_scale_cache"], case["k_scale_cache"])          # the scale tensors are not touched
    assert torch.equal(got["q_norm_scale"], torch.zeros_like(got["q_norm_scale"]))


def test_bf16_form_reference_case_b4_s2(cuda):
    # the reference's test_b4_s64k2_pa_nd_bf16_d: no quantisation anywhere (empty dequant_scale, bf16 w_uq_qr and cache)
    case = op.make_case(4, 2, 1024, seed=18, quant_b=False)
    check_bf16_form(case, run(case, cuda))


def test_bf16_form_small_sizes_and_ragged_token_tiles(cuda):
    for b, s1, seed in ((1, 1, 19), (37, 1, 20)):
        case = op.make_case(b, s1, 300, seed=seed, h=512, q_lora_rank=256, n=4, quant_b=False)
        check_bf16_form(case, run(case, cuda))
    case = op.make_case(3, 2, 300, seed=21, h=1280, q_lora_rank=1280, n=6, quant_b=False)   # ragged last splits
    check_bf16_form(case, run(case, cuda, entry="mla_prolog_quant_p"))


def test_bf16_form_feeds_sparse_flash_attention(cuda):
    """The bf16 cache rows the bf16 form writes are what sparse flash attention reads in its bf16-cache flavour."""
    from _cases import run_sfa
    from test_gpu_sfa import full_check
    b, s1, s2 = 2, 2, 300
    case = op.make_case(b, s1, s2, seed=22, quant_b=False)
    got = run(case, cuda)
    tk = torch.zeros((b * s1, 2048), dtype=torch.int32)
    tk[:, :s2] = torch.arange(s2, dtype=torch.int32)
    ca = {"b": b, "s1": s1, "nq": 128, "topk": 2048, "block_size": 128, "softmax_scale": 192 ** -0.5,
          "act_seq": [s2] * b, "q": torch.cat([got["q_nope"], got["q_rope"]], dim=-1).reshape(b, s1, 128, 576),
          "kn": got["kv_cache"].view(-1, 512), "kr": got["kr_cache"].view(-1, 64),
          "kn_scales": torch.ones((got["kv_cache"].view(-1, 512).shape[0], 4), dtype=torch.float32),
          "topk_indices": tk, "block_table": case["block_table"]}
    full_check(run_sfa(ca, cuda), ca, "bf16 prolog -> attention")


def test_prolog_feeds_sparse_flash_attention(cuda):
    """Stage chaining: the query the prolog writes and the cache rows it adds are, as they are, what sparse flash
    attention reads (int8 kv rows with four fp32 scales, bf16 rope rows, q_nope | q_rope)."""
    from _cases import run_sfa
    from test_gpu_sfa import full_check
    b, s1, s2 = 3, 2, 300
    case = op.make_case(b, s1, s2, seed=16)
    got = run(case, cuda)
    rows = case["cache_index"]
    # the reference generator leaves the old cache rows in whatever range; attention needs them plausible, which they are
    # (int8 rows with positive scales from quant()).  Every position of a sequence is attended, the new ones included.
    tk = torch.zeros((b * s1, 2048), dtype=torch.int32)
    tk[:, :s2] = torch.arange(s2, dtype=torch.int32)
    ca = {"b": b, "s1": s1, "nq": 128, "topk": 2048, "block_size": 128, "softmax_scale": 192 ** -0.5,
          "act_seq": [s2] * b, "q": torch.cat([got["q_nope"], got["q_rope"]], dim=-1).reshape(b, s1, 128, 576),
          "kn": got["kv_cache"].view(-1, 512), "kr": got["kr_cache"].view(-1, 64),
          "kn_scales": got["k_scale_cache"].view(-1, 4), "topk_indices": tk, "block_table": case["block_table"]}
    assert (ca["kn_scales"][rows] > 0).all()
    out = run_sfa(ca, cuda)   # the attention takes the caches as 2-D views [rows, dim], like the reference's driver
    full_check(out, ca, "prolog -> attention")


def test_errors(cuda):
    from pypto_amd.error import FeError
    case = op.make_case(2, 1, 256, seed=1, h=512, q_lora_rank=256, n=4)
    with pytest.raises(FeError, match="int64|INT64"):
        run(dict(case, cache_index=case["cache_index"].int()), cuda)
    with pytest.raises(FeError, match="multiple of 256"):
        run(op.make_case(2, 1, 256, seed=1, h=512, q_lora_rank=384, n=4, quant_b=False), cuda)
    with pytest.raises(FeError, match="int8 form"):     # bf16 weights with a non-empty dequant_scale: neither form
        run(dict(case, w_uq_qr=case["w_uq_qr"].to(torch.bfloat16)), cuda)
    with pytest.raises(FeError, match="heads"):
        run(dict(case, w_uk=case["w_uk"][:3].contiguous(), w_uq_qr=case["w_uq_qr"][:, :576].contiguous(),
                 w_qb_scale=case["w_qb_scale"][:576].contiguous()), cuda)
