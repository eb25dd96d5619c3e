"""GPU parity: fused MLA prolog + lightning-indexer prolog (HIP, through the C ABI).

Two bars.  (1) Plumbing: the fused call must give what the two operators give when called one after the other with the
MLA prolog's q_norm / q_norm_scale handed over by the caller - bit for bit for every MLA output and for the indexer's
query (integer GEMM, same epilogue); the indexer's key path and weights sum x @ [w_k | w_proj] in a different order when
fused (the product rides along in the MLA prolog's first kernel), so there: int8 within 1, fp16 within one bf16 step.
(2) Against the oracle's composition of
the two goldens: the MLA outputs as in test_gpu_mla_prolog; the indexer outputs inherit the (rare, one-step) q_norm
differences of the MLA stage, which is why the reference widens q_int8's tolerance to 2 here
(deepseekv32_mla_indexer_prolog_quant.py:824): int8 within 2 everywhere and equal in at least 95 % of the places, scales
and weights within one bf16 step.
"""
import pytest
import torch

from oracle import mla_prolog as op
from test_gpu_indexer_prolog import WEIGHTS_REL, weights_allowance
from test_gpu_mla_prolog import FEW, check_rope_cache

pytestmark = pytest.mark.gpu
EPS = 1e-5


def _impl():
    from pypto_amd.deepseek_v32_exp import lightning_indexer_prolog_quant_impl as ip
    from pypto_amd.deepseek_v32_exp import mla_indexer_prolog_quant_impl as fused
    from pypto_amd.deepseek_v32_exp import mla_prolog_quant_impl as mla
    return mla, ip, fused


def _buffers(mla_case, idx_case, dev):
    t, r = mla_case["x"].shape[0], mla_case["w_dq"].shape[1]
    n, ni = mla_case["w_uk"].shape[0], idx_case["w_proj"].shape[1]
    m = {k: v.to(dev) for k, v in mla_case.items()}
    i = {k: v.to(dev) for k, v in idx_case.items()}
    z = lambda shape, dt: torch.zeros(shape, dtype=dt, device=dev)  # noqa: E731
    out = {"q_norm": z((t, r), torch.int8), "q_norm_scale": z((t, 1), torch.float32),
           "q_nope": z((t, n, 512), torch.bfloat16), "q_rope": z((t, n, 64), torch.bfloat16),
           "kv_cache": m["kv_cache"].clone(), "kr_cache": m["kr_cache"].clone(), "k_scale_cache": m["k_scale_cache"].clone(),
           "q_int8": z((t, ni, 128), torch.int8), "q_scale": z((t, ni, 1), torch.float16),
           "k_cache": i["k_cache"].clone(), "idx_k_scale_cache": i["k_scale_cache"].clone(),
           "weights": z((t, ni), torch.float16)}
    return m, i, out


def run_fused(mla_case, idx_case, dev, entry="mla_indexer_prolog_quant_d"):
    mla, ip, fused = _impl()
    m, i, o = _buffers(mla_case, idx_case, dev)
    getattr(fused, entry)(
        m["x"], m["w_dq"], m["w_uq_qr"], m["w_qb_scale"], m["w_uk"], m["w_dkv_kr"], m["gamma_cq"], m["gamma_ckv"], m["cos"],
        m["sin"], m["cache_index"], o["kv_cache"], o["kr_cache"], o["k_scale_cache"], i["w_qb"], i["w_qb_scale"], i["w_k"],
        i["w_proj"], i["ln_gamma"], i["ln_beta"], i["hadamard_q"], i["hadamard_k"], o["k_cache"], o["idx_k_scale_cache"],
        o["q_nope"], o["q_rope"], o["kv_cache"], o["kr_cache"], o["k_scale_cache"], o["q_int8"], o["q_scale"], o["k_cache"],
        o["idx_k_scale_cache"], o["weights"], EPS, EPS, "PA_BSND", mla.MlaTileConfig(), ip.IndexerPrologQuantAttr(eps=1e-6),
        ip.IndexerPrologQuantConfigs(), mla.RopeTileShapeConfig([32, 64], [32, 32, 128], [16, 128, 128, 128]))
    torch.cuda.synchronize()
    return {k: v.cpu() for k, v in o.items() if k not in ("q_norm", "q_norm_scale")}


def run_separate(mla_case, idx_case, dev):
    mla, ip, _ = _impl()
    m, i, o = _buffers(mla_case, idx_case, dev)
    mla.mla_prolog_quant_d(
        m["x"], m["w_dq"], m["w_uq_qr"], m["w_qb_scale"], m["w_uk"], m["w_dkv_kr"], m["gamma_cq"], m["gamma_ckv"], m["cos"],
        m["sin"], m["cache_index"], o["kv_cache"], o["kr_cache"], o["k_scale_cache"], o["q_norm"], o["q_norm_scale"],
        o["q_nope"], o["q_rope"], o["kv_cache"], o["kr_cache"], o["k_scale_cache"], EPS, EPS, "PA_BSND", mla.MlaTileConfig(),
        mla.RopeTileShapeConfig([32, 64], [32, 32, 128], [16, 128, 128, 128]))
    ip.lightning_indexer_prolog_quant(
        m["x"], o["q_norm"], o["q_norm_scale"], i["w_qb"], i["w_qb_scale"], i["w_k"], i["w_proj"], i["ln_gamma"],
        i["ln_beta"], m["cos"], m["sin"], i["hadamard_q"], i["hadamard_k"], o["k_cache"], o["idx_k_scale_cache"],
        m["cache_index"], o["q_int8"], o["q_scale"], o["k_cache"], o["idx_k_scale_cache"], o["weights"],
        ip.IndexerPrologQuantConfigs(), ip.IndexerPrologQuantAttr(eps=1e-6))
    torch.cuda.synchronize()
    return {k: v.cpu() for k, v in o.items()}


def check_against_oracle(mla_case, idx_case, got):
    gm, gi = op.mla_indexer_prolog(mla_case, idx_case, EPS, EPS, 1e-6)
    rows = mla_case["cache_index"]

    def ints(a, b, name, tol, min_equal):
        diff = (a.int() - b.int()).abs()
        # (a quantisation scale that moved by one bf16 step of the row's largest value moves a quantised value v by
        # v / 128 steps: in the upper half of the int8 range that is one more step than the value's own rounding)
        assert (diff <= tol + (b.int().abs() >= 64).int()).all(), f"{name}: off by {int(diff.max())}"
        assert (diff == 0).float().mean() >= min_equal, f"{name}: {(diff != 0).float().mean():.4f} of the values differ"

    def close(a, b, name, rel=2.0 ** -7, atol=1e-8, outliers=0.0):
        a, b = a.float().flatten(), b.float().flatten()
        assert torch.isfinite(a).all(), name
        ratio = (a - b).abs() / (rel * b.abs() + atol)
        assert int((ratio > 1).sum()) <= (max(outliers * ratio.numel(), FEW) if outliers else 0) and ratio.max() <= 3, \
            f"{name}: {int((ratio > 1).sum())} values out of tolerance, worst {float(ratio.max())} x"

    ints(got["kv_cache"].view(-1, 512)[rows], gm["kv_cache"].view(-1, 512)[rows], "kv_cache", 1, 0.98)
    close(got["k_scale_cache"].view(-1, 4)[rows], gm["k_scale_cache"].view(-1, 4)[rows], "k_scale_cache", rel=2.0 ** -6)  # see test_gpu_mla_prolog
    close(got["q_nope"], gm["q_nope"], "q_nope", 0.0078125, 0.005, outliers=5e-3)   # see test_gpu_mla_prolog
    close(got["q_rope"], gm["q_rope"], "q_rope", 0.0078125, 0.005, outliers=5e-3)
    check_rope_cache(mla_case, got["kr_cache"], gm["kr_cache"], EPS)   # see test_gpu_mla_prolog
    # (the reference's widened tolerance of 2; with a q_lora_rank of 128 a flipped q_norm value is one of only 128 terms
    # of a product and moves it by more: 3 there)
    ints(got["q_int8"], gi["q_int8"], "q_int8", 2 if mla_case["w_dq"].shape[1] >= 256 else 3, 0.95)
    # (the golden's index queries come from the golden's q_norm, the product's from its own: a q_norm value that rounded
    # the other way shifts the 128 values of a head a little, on top of the one bf16 step their own rounding can move,
    # which is why q_int8 gets 2 above; a query scale follows the largest of them, so two bf16 steps here.  The tight
    # check of this stage is that the fused call gives the bits of the separate calls, whose index prolog is tested
    # against the oracle from one and the same q_norm.)
    close(got["q_scale"], gi["q_scale"], "q_scale", rel=2.0 ** -6)
    ints(got["k_cache"].view(-1, 128)[rows], gi["k_cache"].view(-1, 128)[rows], "idx k_int8", 1, 0.98)
    close(got["idx_k_scale_cache"].view(-1)[rows], gi["k_scale_cache"].view(-1)[rows], "idx k_scale")
    close(got["weights"], gi["weights"], "weights", rel=WEIGHTS_REL, atol=weights_allowance(idx_case).flatten())


def same_as_separate(fused, sep, idx_case):
    for k, v in fused.items():
        if k in ("k_cache", "idx_k_scale_cache", "weights"):
            continue
        assert torch.equal(v, sep[k]), f"{k}: fused and separate calls differ"
    assert (fused["k_cache"].int() - sep["k_cache"].int()).abs().max() <= 1
    assert (fused["k_cache"] == sep["k_cache"]).float().mean() >= 0.999
    a, b = fused["idx_k_scale_cache"].float(), sep["idx_k_scale_cache"].float()
    assert ((a - b).abs() <= 2.0 ** -7 * b.abs() + 1e-8).all(), "idx_k_scale_cache"
    # weights near zero are sums that cancel: there the summation order shows at the fp32 level of the h terms
    a, b = fused["weights"].float(), sep["weights"].float()
    assert ((a - b).abs() <= WEIGHTS_REL * b.abs() + weights_allowance(idx_case)).all(), "weights"


def test_reference_case_b4_s2_fused_equals_separate_and_oracle(cuda):
    # the reference's enabled test test_b_4_s1_2_tilebs_8_d: b=4, two new tokens per sequence, model sizes
    mla_case, idx_case = op.make_fused_case(4, 2, 1024, seed=21)
    fused = run_fused(mla_case, idx_case, cuda)
    sep = run_separate(mla_case, idx_case, cuda)
    same_as_separate(fused, sep, idx_case)
    check_against_oracle(mla_case, idx_case, fused)


def test_prefill_entry_ragged_tiles_small_sizes(cuda):
    mla_case, idx_case = op.make_fused_case(37, 1, 300, seed=22, n_idx=64, h=512, q_lora_rank=256, n=4)
    fused = run_fused(mla_case, idx_case, cuda, entry="mla_indexer_prolog_quant_p")
    sep = run_separate(mla_case, idx_case, cuda)
    same_as_separate(fused, sep, idx_case)
    check_against_oracle(mla_case, idx_case, fused)


def test_prefill_sizes_fused_equals_separate_and_oracle(cuda):
    # 128 tokens and more: the first product of both calls runs the kernel that owns an output tile, and so does the
    # separate call's int8 product (exact, so still the fused call's bits)
    # (up to 256 tokens the two int8 products of the fused call share a launch, above they are launches of their own)
    for b, seed in ((150, 24), (300, 25)):
        mla_case, idx_case = op.make_fused_case(b, 1, 300, seed=seed, n_idx=64, h=1280, q_lora_rank=256, n=4)
        fused = run_fused(mla_case, idx_case, cuda, entry="mla_indexer_prolog_quant_p")
        sep = run_separate(mla_case, idx_case, cuda)
        same_as_separate(fused, sep, idx_case)
        check_against_oracle(mla_case, idx_case, fused)


def test_index_head_counts_without_the_side_by_side_kernels(cuda):
    # 32 index heads: x @ w_proj is half an output tile wide, so the fused entry runs the two operators back to back
    mla_case, idx_case = op.make_fused_case(5, 1, 300, seed=23, n_idx=32, h=512, q_lora_rank=256, n=4)
    fused = run_fused(mla_case, idx_case, cuda)
    sep = run_separate(mla_case, idx_case, cuda)
    for k, v in fused.items():
        assert torch.equal(v, sep[k]), f"{k}: fused and separate calls differ"


def test_decode_layer_front_end_chain(cuda):
    """One decode layer's attention front end as three chained calls on the GPU, each stage checked against the oracle
    on the previous stage's actual outputs: fused prolog -> (indexer query, weights, updated index cache) -> lightning
    indexer -> top-k rows -> sparse flash attention over the updated int8 MLA cache with the prolog's query."""
    from _cases import run_indexer, run_sfa
    from test_gpu_indexer import check_topk
    from test_gpu_sfa import full_check
    b, s1, s2 = 2, 2, 3000
    mla_case, idx_case = op.make_fused_case(b, s1, s2, seed=25)
    got = run_fused(mla_case, idx_case, cuda)
    n_pages = got["k_cache"].shape[0]
    ci = {"query": got["q_int8"], "q_scale": got["q_scale"].reshape(b * s1, 64), "weights": got["weights"],
          "key_cache": got["k_cache"], "k_scale": got["idx_k_scale_cache"].reshape(n_pages, 128, 1),
          "act_seq": [s2] * b, "block_table": mla_case["block_table"], "b": b, "s1": s1, "selected_count": 2048,
          "block_size": 128}
    topk = run_indexer(ci, cuda)
    check_topk(ci, topk)
    ca = {"b": b, "s1": s1, "nq": 128, "topk": 2048, "block_size": 128, "softmax_scale": 192 ** -0.5, "act_seq": [s2] * b,
          "q": torch.cat([got["q_nope"], got["q_rope"]], dim=-1).reshape(b, s1, 128, 576),
          "kn": got["kv_cache"].view(-1, 512), "kr": got["kr_cache"].view(-1, 64),
          "kn_scales": got["k_scale_cache"].view(-1, 4), "topk_indices": topk.reshape(b * s1, 2048),
          "block_table": mla_case["block_table"]}
    # the newest token of a query's causal range is its own, just-written cache row: it must be reachable
    new_rows = mla_case["cache_index"].reshape(b, s1)
    assert (ca["kn_scales"][new_rows.reshape(-1)] > 0).all()
    full_check(run_sfa(ca, cuda), ca, "prolog -> indexer -> attention")


def test_no_tokens_is_a_no_op(cuda):
    """An empty batch (t = 0) is accepted by all three prolog entries and touches nothing."""
    mla_case, idx_case = op.make_fused_case(2, 1, 256, seed=24, n_idx=64, h=512, q_lora_rank=256, n=4)
    for k in ("x", "cos", "sin", "cache_index"):
        mla_case[k] = mla_case[k][:0].contiguous()
    idx_case.update(x=mla_case["x"], cos=mla_case["cos"], sin=mla_case["sin"], k_cache_index=mla_case["cache_index"])
    fused = run_fused(mla_case, idx_case, cuda)
    sep = run_separate(mla_case, idx_case, cuda)
    for got in (fused, sep):
        assert torch.equal(got["kv_cache"], mla_case["kv_cache"]) and torch.equal(got["kr_cache"], mla_case["kr_cache"])
        assert torch.equal(got["k_scale_cache"], mla_case["k_scale_cache"])
        assert torch.equal(got["k_cache"], idx_case["k_cache"])
        assert torch.equal(got["idx_k_scale_cache"], idx_case["k_scale_cache"])
        assert got["q_nope"].shape == (0, 4, 512) and got["q_int8"].shape == (0, 64, 128)


def test_errors(cuda):
    from pypto_amd.error import FeError
    mla_case, idx_case = op.make_fused_case(2, 1, 256, seed=1, n_idx=32, h=512, q_lora_rank=256, n=4)
    with pytest.raises(FeError, match="heads"):
        run_fused(mla_case, dict(idx_case, w_proj=idx_case["w_proj"][:, :16].contiguous()), cuda)
    with pytest.raises(FeError, match="int64|INT64"):
        run_fused(dict(mla_case, cache_index=mla_case["cache_index"].int()), idx_case, cuda)
