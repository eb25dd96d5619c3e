"""GPU parity: lightning-indexer prolog (HIP, through the C ABI) against the CPU oracle.

Bar.  The reference compares int8 outputs with an absolute tolerance of 1 and the fp16 scales and weights with 2.5e-5
(deepseekv32_lightning_indexer_prolog_quant.py:378-382).  Every stage here reproduces the golden's rounding points;
what differs is the summation order of the two fp32 matmuls (7168 and 128 terms), which now and then moves a value
across a bf16 rounding boundary before the quantisation.  So: int8 values within 1 everywhere and equal in at least
98 % of the places; scales within one bf16 step (2^-7 relative) everywhere and bit-equal in at least 90 % of the rows;
weights within one bf16 step and bit-equal in at least 98 % of the places.
"""
import pytest
import torch

from oracle import indexer_prolog as op

pytestmark = pytest.mark.gpu


def run(case, dev):
    from pypto_amd.deepseek_v32_exp import lightning_indexer_prolog_quant_impl as impl
    t = case["x"].shape[0]
    n = case["w_proj"].shape[1]
    d = {k: v.to(dev) for k, v in case.items()}
    inp = impl.IndexerPrologQuantInput(
        x=d["x"], q_norm=d["q_norm"], q_norm_scale=d["q_norm_scale"], w_qb=d["w_qb"], w_qb_scale=d["w_qb_scale"],
        wk=d["w_k"], w_proj=d["w_proj"], ln_gamma_k=d["ln_gamma"], ln_beta_k=d["ln_beta"], cos_idx_rope=d["cos"],
        sin_idx_rope=d["sin"], hadamard_q=d["hadamard_q"], hadamard_k=d["hadamard_k"], k_cache=d["k_cache"].clone(),
        k_cache_scale=d["k_scale_cache"].clone(), k_cache_index=d["k_cache_index"])
    out = impl.IndexerPrologQuantOutput(
        q_int8=torch.zeros((t, n, 128), dtype=torch.int8, device=dev),
        q_scale=torch.zeros((t, n, 1), dtype=torch.float16, device=dev),
        k_int8=inp.k_cache, k_scale=inp.k_cache_scale,
        weights=torch.zeros((t, n), dtype=torch.float16, device=dev))
    tensors = list(vars(inp).values()) + list(vars(out).values())
    impl.lightning_indexer_prolog_quant(*tensors, impl.IndexerPrologQuantConfigs(), impl.IndexerPrologQuantAttr(eps=1e-6))
    torch.cuda.synchronize()
    return {"q_int8": out.q_int8.cpu(), "q_scale": out.q_scale.cpu(), "k_cache": out.k_int8.cpu(),
            "k_scale_cache": out.k_scale.cpu(), "weights": out.weights.cpu()}


WEIGHTS_REL = 2.0 ** -7 + 2.0 ** -10   # one bf16 step at the bottom of a binade, and an fp16 rounding (up to 2^-11) on either side


def weights_allowance(case):
    """What the summation order of x @ w_proj (h fp32 terms) may move a weight by, in the weight's units: a weight is
    that sum times 1 / sqrt(heads * 128), and where the terms cancel the sum carries an absolute error of a few units in
    the last place of the terms' magnitudes, whatever the order - 8 * 2^-24 * sum |x_i| |w_i| is a generous bound for
    the blocked orders of either side.  Both the kernel and the golden sit within it of the exact sum, so twice that."""
    n = case["w_qb"].shape[1] // case["hadamard_q"].shape[0]
    mag = case["x"].double().abs() @ case["w_proj"].double().abs()
    return (2 * 8 * 2.0 ** -24 * mag * (n * case["hadamard_q"].shape[0]) ** -0.5).float()


def check(case, got):
    gold = op.indexer_prolog(case)
    rows = case["k_cache_index"]

    def ints(a, b, name):
        diff = (a.int() - b.int()).abs()
        assert diff.max() <= 1, f"{name}: off by {int(diff.max())}"
        assert (diff == 0).float().mean() >= 0.98, f"{name}: {(diff != 0).float().mean():.4f} of the values differ"

    def scales(a, b, name, min_equal, atol=1e-8, rel=2.0 ** -7):
        a, b = a.float().flatten(), b.float().flatten()
        assert torch.isfinite(a).all(), name
        assert ((a - b).abs() <= rel * b.abs() + atol).all(), f"{name}: {float(((a - b).abs() / b.abs()).max())}"
        assert (a == b).float().mean() >= min_equal, f"{name}: only {(a == b).float().mean():.3f} bit-equal"

    ints(got["q_int8"], gold["q_int8"], "q_int8")
    # (fp16 scales: one bf16 step of the row's largest value plus the two fp16 roundings, like the weights below)
    scales(got["q_scale"], gold["q_scale"], "q_scale", 0.90, rel=WEIGHTS_REL)
    ints(got["k_cache"].view(-1, 128)[rows], gold["k_cache"].view(-1, 128)[rows], "k_int8")
    scales(got["k_scale_cache"].view(-1)[rows], gold["k_scale_cache"].view(-1)[rows], "k_scale", 0.80, rel=WEIGHTS_REL)
    # (a weight is the bf16 rounding of the sum, scaled and rounded to fp16: a sum that rounds the other way moves it by
    # one bf16 step, 2^-7 of the value at the bottom of a binade, and the two fp16 roundings add up to 2^-11 each)
    scales(got["weights"], gold["weights"], "weights", 0.98, atol=weights_allowance(case).flatten(), rel=WEIGHTS_REL)
    # nothing but the indexed rows of the caches may change
    keep = torch.ones(case["k_cache"].shape[0] * case["k_cache"].shape[1], dtype=torch.bool)
    keep[rows] = False
    assert torch.equal(got["k_cache"].view(-1, 128)[keep], case["k_cache"].view(-1, 128)[keep])
    assert torch.equal(got["k_scale_cache"].view(-1)[keep], case["k_scale_cache"].view(-1)[keep])


def test_reference_case_b4_s1_2(cuda):
    # the reference's enabled test: b=4, two new tokens per sequence, model sizes (h 7168, q_lora_rank 1536, 64 x 128)
    case = op.make_case(4, 2, 4096, seed=7)
    check(case, run(case, cuda))


def test_decode_batch_and_ragged_token_tiles(cuda):
    for b, s1, seed in ((32, 1, 8), (37, 1, 9), (128, 4, 10), (1, 1, 11)):
        case = op.make_case(b, s1, 1024, seed=seed)
        check(case, run(case, cuda))


def test_prefill_sizes_same_bits_as_the_decode_kernels(cuda):
    """From 128 tokens on the query product runs per (head, 128 tokens) instead of per (head, 32 tokens), beside the x
    product per 128 tokens.  Its integer
    sums are exact and the rest is the same arithmetic, so the query outputs must be the bits the decode-size kernels
    give for the same tokens (run here in slices of fewer than 128 tokens) - on token counts that leave ragged tiles."""
    for b, s1, seed in ((64, 2, 20), (75, 4, 21), (257, 1, 22), (199, 1, 23)):
        case = op.make_case(b, s1, 1024, seed=seed)
        got = run(case, cuda)
        check(case, got)
        t = b * s1
        per_token = ("x", "q_norm", "q_norm_scale", "cos", "sin", "k_cache_index")
        for t0 in range(0, t, 100):
            part = {k: (v[t0:t0 + 100] if k in per_token else v) for k, v in case.items()}
            small = run(part, cuda)
            assert torch.equal(small["q_int8"], got["q_int8"][t0:t0 + 100]), (t, t0)
            assert torch.equal(small["q_scale"], got["q_scale"][t0:t0 + 100]), (t, t0)


def test_walsh_hadamard_and_other_sizes(cuda):
    case = op.make_case(3, 2, 512, seed=12, hadamard="walsh")
    check(case, run(case, cuda))
    case = op.make_case(5, 1, 300, seed=13, h=1024, q_lora_rank=256, n=32)
    check(case, run(case, cuda))


def test_prolog_feeds_the_indexer(cuda):
    """Stage chaining: the prolog's outputs are, as they are, the lightning indexer's inputs (query, query scale,
    weights, the updated paged key cache and its scale cache)."""
    from oracle import indexer as oi
    from test_gpu_indexer import check_topk
    from _cases import run_indexer
    b, s1, s2 = 3, 2, 3000
    case = op.make_case(b, s1, s2, seed=14)
    # the reference generator's key scales are U[-1,1); the indexer takes any sign, keep them as they are
    got = run(case, cuda)
    ci = {"query": got["q_int8"], "q_scale": got["q_scale"].reshape(b * s1, 64), "weights": got["weights"],
          "key_cache": got["k_cache"], "k_scale": got["k_scale_cache"].reshape(got["k_cache"].shape[0], 128, 1),
          "act_seq": [s2] * b, "block_table": case["block_table"], "b": b, "s1": s1, "selected_count": 2048,
          "block_size": 128}
    check_topk(ci, run_indexer(ci, cuda))


def test_errors(cuda):
    from pypto_amd.error import FeError
    case = op.make_case(2, 1, 256, seed=1, h=512, q_lora_rank=128, n=32)
    bad = dict(case, k_cache_index=case["k_cache_index"].int())
    with pytest.raises(FeError, match="int64"):
        run(bad, cuda)
    bad = dict(case, w_proj=case["w_proj"][:, :16].contiguous())
    with pytest.raises(FeError, match="heads"):
        run(bad, cuda)
