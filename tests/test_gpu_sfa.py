"""GPU parity: sparse flash attention (HIP, through the C ABI) against the CPU oracle."""
import pytest
import torch

from oracle import sfa as osfa
from oracle.compare import compare, count_violations

from _cases import run_sfa, sfa_golden

pytestmark = pytest.mark.gpu

# BASELINE bar: within 2e-2 relative / 1e-2 absolute in bf16 (no element may exceed it);
# the reference's own bar: at most 0.5 % of elements outside 1e-4 + 5e-3 * |ref|.
ABS_TOL, REL_TOL = 1e-2, 2e-2


def check(out, gold, name, strict=True):
    assert not torch.isnan(out).any() and not torch.isinf(out).any(), name
    assert count_violations(out, gold, ABS_TOL, REL_TOL) == 0, name
    if strict:
        compare(out, gold, name, atol=1e-4, rtol=5e-3)


def check_vs_fp64(out, case, golds, name):
    """Where the softmax is peaked the reference's goldens differ from each other by bf16 rounding of P
    (no-flash vs flash disagree on ~18 % of elements under the strict comparator), so the strict comparator
    cannot hold against either; instead the kernel must be as close to float64 attention as they are."""
    ref = osfa.attention_fp64(case["q"], case["kn"], case["kr"], case["kn_scales"], case["topk_indices"],
                              case["block_table"], case["act_seq"], case["block_size"], case["softmax_scale"],
                              case["topk"])
    err = float((out.double() - ref).abs().max())
    gold_err = max(float((g.double() - ref).abs().max()) for g in golds)
    assert err <= 1.5 * gold_err + 1e-6, f"{name}: max error {err} vs golden's own {gold_err}"
    bad = count_violations(out.double(), ref, 1e-4, 5e-3) / ref.numel()
    gold_bad = max(count_violations(g.double(), ref, 1e-4, 5e-3) / ref.numel() for g in golds)
    assert bad <= 1.5 * gold_bad + 0.005, f"{name}: {bad} of elements off vs golden's own {gold_bad}"


def test_tiny_config1(cuda):
    # b=1, 16 heads, 4096-token cache, top-256, scale 1/sqrt(192)
    case = osfa.make_case(1, 16, 1, [4096], topk=256, seed=7, dist="bench", softmax_scale=192 ** -0.5)
    out = run_sfa(case, cuda)
    g0, g1 = sfa_golden(case), sfa_golden(case, flash=True, s2_tile=64)
    check(out, g0, "config1 vs no-flash golden", strict=False)
    check(out, g1, "config1 vs flash golden", strict=False)
    check_vs_fp64(out, case, [g0, g1], "config1")


def test_tiny_reference_distribution(cuda):
    # same shape on the reference generator's distribution (U[-1,1), scale 576^-0.5)
    case = osfa.make_case(1, 16, 1, [4096], topk=256, seed=11)
    out = run_sfa(case, cuda)
    g0, g1 = sfa_golden(case), sfa_golden(case, flash=True, s2_tile=64)
    check(out, g0, "config1-uniform vs no-flash golden", strict=False)
    check(out, g1, "config1-uniform vs flash golden", strict=False)
    check_vs_fp64(out, case, [g0, g1], "config1-uniform")


@pytest.mark.parametrize("packed", [False, True])
def test_reference_case_mixed_lengths(cuda, packed):
    # the reference's decode test case: (b, nq, nkv, s1) = (4, 128, 1, 2), lengths 65536 / 16381 / 666 / 15
    case = osfa.make_case(4, 128, 2, [65536, 16381, 666, 15], seed=42)
    out = run_sfa(case, cuda, packed=packed)
    g0 = sfa_golden(case)
    check(out, g0, "mixed lengths vs no-flash golden", strict=False)
    check_vs_fp64(out, case, [g0], "mixed lengths")
    # sequences 2 and 3 are shorter than s1 + topk: rows past cur_seq must not matter, row (3, 0) has cur_seq 14
    assert out.shape == (4, 2, 128, 512)
