"""GPU parity: lightning indexer (HIP, through the C ABI) against the CPU oracle.

Bar: top-k indices bit-exact wherever score gaps exceed fp32 summation tolerance.  The golden's 64-term head sum
is an fp32 BLAS reduction whose order is unspecified, so two scores closer than a few fp32 ulps of the row's
largest score may legitimately swap; everything else must match the golden slot for slot, including the -1
padding and the ascending-index order of exactly equal scores.
"""
import pytest
import torch

from oracle import indexer as oi
from oracle.compare import topk_idx_compare

from _cases import indexer_scores, run_indexer
from _fixtures import load_indexer_small

pytestmark = pytest.mark.gpu


def check_topk(case, got, exact=None, strict_ties=False):
    """strict_ties: equal golden scores must come in ascending index order.  Only valid where equal scores come from
    identical key rows (then the kernel's fp32 sums are bit-identical too); two different keys whose exact scores
    happen to coincide may differ by an ulp in the kernel's summation order and then fall under the tolerance rule."""
    s1, k = case["s1"], case["selected_count"]
    if exact is None:
        exact = indexer_scores(case, exact=True)
    gold = oi.select(indexer_scores(case), case["act_seq"], s1, k)
    swaps = 0
    for r in range(got.shape[0]):
        n = max(oi.eff_seq_of(case["act_seq"][r // s1], s1, r % s1), 0)
        kk = min(n, k)
        row = got[r, 0]
        assert (row[kk:] == -1).all(), f"row {r}: padding"
        sel = row[:kk].long()
        assert ((sel >= 0) & (sel < max(n, 1))).all(), f"row {r}: index out of range"
        assert sel.unique().numel() == kk, f"row {r}: duplicates"
        sc = exact[r, :n]
        tol = 1e-5 * float(sc.abs().max()) if n else 0.0
        chosen = sc[sel]
        assert (chosen[:-1] >= chosen[1:] - tol).all(), f"row {r}: not sorted"
        if strict_ties:
            eq = chosen[:-1] == chosen[1:]
            assert (sel[:-1][eq] < sel[1:][eq]).all(), f"row {r}: equal scores must come in ascending index order"
        if n > kk:
            rest = torch.ones(n, dtype=torch.bool)
            rest[sel] = False
            assert float(chosen.min()) >= float(sc[rest].max()) - tol, f"row {r}: a better token was left out"
        for j in (row != gold[r, 0]).nonzero().flatten().tolist():
            a, e = int(row[j]), int(gold[r, 0, j])
            assert a >= 0 and e >= 0 and abs(float(sc[a]) - float(sc[e])) <= tol, f"row {r} slot {j}: {a} vs {e}"
            swaps += 1
    # the reference's own comparator: it allows int(k * 5e-4) ids per row to differ, one at the reference's k = 2048
    # (a near-tie at the selection boundary); smaller selections get the same allowance of one
    topk_idx_compare(got, gold, "topk_res", max(5e-4, 1.5 / k), k)
    return swaps


def test_small_edge_lengths(cuda):
    case = oi.make_case(4, 1, [4096, 971, 2048, 15], seed=3)
    check_topk(case, run_indexer(case, cuda))


def test_fp32_scales(cuda):
    """Benchmark configuration 3 as written - fp32 per-token scales - through the same entry point: both score kernels
    (128-token pages and a page size that is not a multiple of 128), one and two query tokens per sequence."""
    for b, s1, act, bs, seed in ((3, 1, [9000, 2049, 300], 128, 61), (2, 2, [5000, 77], 128, 62), (2, 1, [3000, 500], 48, 63)):
        case = oi.make_case(b, s1, act, block_size=bs, seed=seed, scale_dtype=torch.float32)
        check_topk(case, run_indexer(case, cuda))
    # one fp16 and one fp32 scale tensor is neither form
    from pypto_amd.error import FeError
    with pytest.raises(FeError, match="idx_key_scale"):
        run_indexer(dict(case, k_scale=case["k_scale"].half()), cuda)


def test_fp32_scale_products_round_twice_like_the_golden(cuda):
    """fp16(fp32(scale * weight)) rounds twice; a fused multiply-convert would round the exact product once and land on
    another fp16 value about once in 8000 products.  Every (token, head) here is such a pair (found by search), so a
    kernel that rounds once gets every per-head factor wrong by an ulp and fails the ordering check."""
    g = torch.Generator().manual_seed(81)
    a = (0.005 + 0.015 * torch.rand(8000000, generator=g)).float()
    w = (torch.randn(8000000, generator=g) / 8).half()
    twice = (a * w.float()).half()
    # (numpy rounds float64 to float16 in one step; torch goes through float32)
    once = torch.from_numpy((a.double().numpy() * w.double().numpy()).astype("float16"))
    hit = (twice != once).nonzero().flatten()
    assert hit.numel() >= 4 * 64
    for bs in (128, 48):
        case = oi.make_case(2, 2, [3000, 500], block_size=bs, seed=82, scale_dtype=torch.float32)
        case["q_scale"] = a[hit[:256]].reshape(4, 64).clone()
        case["weights"] = w[hit[:256]].reshape(4, 64).clone()
        assert not torch.equal(oi.w_scale_of(case["q_scale"], case["weights"]), once[hit[:256]].reshape(4, 64))
        check_topk(case, run_indexer(case, cuda))


def test_scores_outside_the_histogram_range(cuda):
    """The selection histogram resolves magnitudes 2^-20 .. 2^12; smaller and larger scores share the first and last bin
    of their sign, whose keys do not share a bit prefix.  fp32 scales put whole rows out of range: tiny scores (the
    threshold bin is a first bin - once with a tie list that fits LDS, once with one that overflows into the pass over
    the whole row), huge scores (a last bin), and a mix of tiny, ordinary and huge ones in one row."""
    for act, qmul, kmul, seed in (([5000, 2300], 1e-5, 1e-5, 71), ([40000], 1e-5, 1e-5, 72), ([9000, 4000], 1e3, 1e3, 73)):
        case = oi.make_case(len(act), 1, act, seed=seed, scale_dtype=torch.float32)
        case["q_scale"] = case["q_scale"] * qmul
        case["k_scale"] = case["k_scale"] * kmul
        sc = indexer_scores(case, exact=True)
        big = sc.abs().max()
        assert (big < 2.0 ** -20) if qmul < 1 else (big > 2.0 ** 12)
        check_topk(case, run_indexer(case, cuda))
    case = oi.make_case(2, 2, [7000, 3000], seed=74, scale_dtype=torch.float32)
    g = torch.Generator().manual_seed(74)
    case["k_scale"] = case["k_scale"] * torch.tensor([1e-9, 1.0, 1e7])[torch.randint(0, 3, case["k_scale"].shape, generator=g)]
    check_topk(case, run_indexer(case, cuda))


def test_mtp_two_query_tokens(cuda):
    case = oi.make_case(4, 2, [5000, 971, 2049, 300], seed=4, dist="driver")
    check_topk(case, run_indexer(case, cuda))


@pytest.mark.parametrize("s1", [1, 3, 4])
def test_query_tokens_per_sequence(cuda, s1):
    case = oi.make_case(3, s1, [2600, 130, 2050], seed=10 + s1)
    check_topk(case, run_indexer(case, cuda))


def test_golden_fixture_with_engineered_ties(cuda):
    case, topk, scores = load_indexer_small()
    got = run_indexer(case, cuda)
    check_topk(case, got, exact=scores, strict_ties=True)
    assert torch.equal(got, topk), "fixture: identical to the oracle slot for slot (gaps far above fp32 noise)"


def test_all_scores_equal_keeps_the_first_indices(cuda):
    # identical keys everywhere: every score ties, the tie list overflows its LDS capacity and the kernel falls back
    # to selecting over the whole row; the rule (ascending index) then fixes the answer completely
    case = oi.make_case(2, 1, [20000, 3000], seed=6)
    case["key_cache"][:] = case["key_cache"][0, 0]
    case["k_scale"][:] = case["k_scale"][0, 0]
    got = run_indexer(case, cuda)
    want = torch.arange(2048, dtype=torch.int32)
    assert torch.equal(got[0, 0], want) and torch.equal(got[1, 0], want)


def test_all_scores_zero(cuda):
    # relu kills every head: scores are +0 / -0, which the ordering must treat as equal
    case = oi.make_case(1, 2, [5000], seed=7)
    case["key_cache"] = -case["query"][0:1, 0:1].reshape(1, 1, 1, 128).expand_as(case["key_cache"]).contiguous()
    case["query"][:] = case["query"][0, 0]
    sc = indexer_scores(case)
    assert (sc[:, :4999] == 0).all()
    got = run_indexer(case, cuda)
    assert torch.equal(got[0, 0], torch.arange(2048, dtype=torch.int32))
    assert torch.equal(got[1, 0], torch.arange(2048, dtype=torch.int32))


def test_reference_cases(cuda):
    # the reference's two decode cases, lengths 64K / 971 / 32K+101 / 16K-1 and the 8-batch one up to 129090 tokens
    for act in ([65536, 971, 32869, 16383], [32767, 32656, 384, 2000, 65536, 971, 32869, 129090]):
        case = oi.make_case(len(act), 2, act, seed=len(act), dist="driver")
        check_topk(case, run_indexer(case, cuda))


def test_contexts_beyond_131072_tokens(cuda):
    case = oi.make_case(2, 1, [140000, 3000], seed=21)
    check_topk(case, run_indexer(case, cuda))
    case = oi.make_case(1, 2, [133000], seed=22, dist="driver")
    check_topk(case, run_indexer(case, cuda))


def test_full_size_config3(cuda):
    # benchmark configuration 3: b=32, 64x128 index heads, context lengths U[8192, 65536], top-2048
    g = torch.Generator().manual_seed(33)
    act = torch.randint(8192, 65537, (32,), generator=g).tolist()
    case = oi.make_case(32, 1, act, seed=33)
    swaps = check_topk(case, run_indexer(case, cuda))
    assert swaps <= 32 * 4, f"{swaps} near-tie swaps"


def test_empty_sequences_and_empty_page_table(cuda):
    # no key anywhere: the cache has no block and the page table no column; every slot is -1
    for s1, bs, k in ((1, 256, 512), (3, 128, 512), (2, 16, 64)):
        case = oi.make_case(1, s1, [0], seed=15, block_size=bs, selected_count=k, dist="driver")
        assert case["block_table"].shape[1] == 0 and case["key_cache"].shape[0] == 0
        got = run_indexer(case, cuda)
        assert (got == -1).all()
        check_topk(case, got)
    # an empty sequence beside a live one
    case = oi.make_case(3, 2, [0, 700, 1], seed=16)
    check_topk(case, run_indexer(case, cuda))


def test_length_beyond_the_page_tables_reach_is_cut_to_it(cuda):
    # act_seq says more tokens than the page table has entries for: keys past the table do not exist, so the answer
    # is the oracle's on the length cut to the table's reach - and no score slot the score kernels never wrote is read
    for s1, bs in ((1, 128), (2, 128), (2, 48)):
        case = oi.make_case(3, s1, [5000, 700, 2500], seed=31 + s1, block_size=bs)
        reach = case["block_table"].shape[1] * bs
        claimed = dict(case, act_seq=[5000 + 70000, 700, 2500])  # (sequence 0 owns every column of the table)
        cut = dict(case, act_seq=[min(a, reach) for a in claimed["act_seq"]])
        got = run_indexer(claimed, cuda)
        assert torch.equal(got, run_indexer(cut, cuda))
        check_topk(cut, got)


def test_cache_without_pages_under_a_page_table(cuda):
    # no page in the cache but a page table with columns and positive lengths: nothing can be addressed, every slot
    # is -1, and no kernel touches the (null) cache
    case = oi.make_case(2, 2, [300, 40], seed=35)
    case["key_cache"] = case["key_cache"][:0].contiguous()
    case["k_scale"] = case["k_scale"][:0].contiguous()
    assert (run_indexer(case, cuda) == -1).all()


def test_coincident_scores_of_different_keys(cuda):
    # the reference generator's small integers make different keys tie exactly in the golden; the kernel may order such
    # a pair either way (its fp32 sum runs in another order), which the tolerance rule of check_topk admits
    case = oi.make_case(1, 2, [7421], seed=1985, dist="driver")
    check_topk(case, run_indexer(case, cuda))


def test_wide_page_table_many_sequences(cuda):
    # 300 short sequences under a page table wide enough for 112 K tokens: 300 x 55 spans of 2048 keys, more than the
    # score kernel's span list holds, so its workgroups take their spans by grid place; and the same sequences under a
    # narrower table, where the list is used and most of its grid has no work
    g = torch.Generator().manual_seed(41)
    act = torch.randint(1, 700, (300,), generator=g).tolist()
    case = oi.make_case(300, 1, act, seed=41, selected_count=64)
    gold_scores = indexer_scores(case, exact=True)
    narrow = run_indexer(case, cuda)
    check_topk(case, narrow, exact=gold_scores)
    bt = case["block_table"]
    wide = dict(case)
    wide["block_table"] = torch.cat([bt, torch.full((bt.shape[0], 880 - bt.shape[1]), -1, dtype=bt.dtype)], dim=1).contiguous()
    assert torch.equal(run_indexer(wide, cuda), narrow)


def test_other_selection_sizes_and_block_sizes(cuda):
    case = oi.make_case(2, 1, [1000, 70], seed=8, selected_count=64)
    check_topk(case, run_indexer(case, cuda))
    case = oi.make_case(2, 2, [1000, 600], seed=9, block_size=48, selected_count=512)  # not a power of two
    check_topk(case, run_indexer(case, cuda))


def test_indexer_feeds_attention(cuda):
    """Stage chaining: the slots the indexer pads with -1 are exactly the slots attention ignores."""
    from oracle import sfa as osfa
    from _cases import run_sfa, sfa_golden
    from oracle.compare import count_violations
    act = [3000, 700, 2048]
    ci = oi.make_case(3, 2, act, seed=15)
    tk = run_indexer(ci, cuda)
    cs = osfa.make_case(3, 128, 2, act, topk=2048, seed=15, dist="bench", softmax_scale=192 ** -0.5)
    cs["topk_indices"] = tk.reshape(6, 2048).clone()
    for r in range(6):
        n = osfa.cur_seq_of(act[r // 2], 2, r % 2, 2048)
        assert (cs["topk_indices"][r, :n] >= 0).all() and (cs["topk_indices"][r, n:] == -1).all()
    out = run_sfa(cs, cuda)
    assert count_violations(out, sfa_golden(cs), 1e-2, 2e-2) == 0


def test_graph_capture_and_replay(cuda):
    from pypto_amd.deepseek_v32_exp import lightning_indexer_quant_impl as impl
    case = oi.make_case(2, 1, [9000, 500], seed=17)
    dev = cuda
    ts = [case["query"].to(dev), case["q_scale"].to(dev), case["key_cache"].to(dev), case["k_scale"].to(dev),
          case["weights"].to(dev), torch.tensor(case["act_seq"], dtype=torch.int32, device=dev),
          case["block_table"].to(dev)]
    eager = run_indexer(case, cuda)
    out = torch.zeros((2, 1, 2048), dtype=torch.int32, device=dev)
    args = ([1], impl.LightningIndexerConfigs(), 2048)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        impl.lightning_indexer_decode(*ts, out, *args)
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        impl.lightning_indexer_decode(*ts, out, *args)
    for _ in range(3):
        out.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out.cpu(), eager)
