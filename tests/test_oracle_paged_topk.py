"""Pins oracle.paged / oracle.topk / oracle.compare against the known answers the reference holds."""
import numpy as np
import pytest
import torch

from oracle import paged
from oracle.compare import compare, topk_idx_compare
from oracle.topk import topk_rows, topk_sorted_stable


def test_gather_docstring_example():
    # python/pypto/experimental/gather.py:57-82: 6x4 table, indices [0,4,3], page table [0,2,1], block size 2
    src = torch.tensor([[10 * r + c for c in range(4)] for r in range(6)], dtype=torch.float16)
    out = paged.paged_gather(src, [0, 4, 3], [0, 2, 1], 2)
    assert out.tolist() == [[0, 1, 2, 3], [20, 21, 22, 23], [50, 51, 52, 53]]


def test_gather_st_case_by_brute_force():
    # python/tests/st/operation/vector/test_gatherinub.py:83-130,205-229: buffer[tok, h] = 10*tok + h (fp16, 32x4),
    # block size 4, 3 logical blocks, page table from Generator seed 42, 8 indices from seed 123
    buf = torch.tensor([[10.0 * t + h for h in range(4)] for t in range(32)], dtype=torch.float16)
    g = torch.Generator().manual_seed(42)
    page = torch.randint(0, 32 // 4, (1, 3), generator=g, dtype=torch.int32)
    g = torch.Generator().manual_seed(123)
    idx = torch.randint(0, 3 * 4, (1, 8), generator=g, dtype=torch.int32)
    out = paged.paged_gather(buf, idx, page[0], 4)
    for j in range(8):
        i = int(idx[0, j])
        phys = int(page[0, i // 4]) * 4 + i % 4
        assert out[j].tolist() == [10.0 * phys + h for h in range(4)]


def test_gather_bounds_are_checked():
    src = torch.zeros((8, 2))
    with pytest.raises(IndexError):
        paged.paged_gather(src, [6], [0, 1, 2], 2)  # logical index beyond the page table
    with pytest.raises(IndexError):
        paged.paged_gather(src, [2], [0, -1], 2)  # unused page
    with pytest.raises(IndexError):
        paged.paged_gather(src, [0], [7], 2)  # physical row outside the cache


def test_block_table_is_a_partition():
    total, table = paged.gen_block_table([300, 5, 128, 129], 128, generator=torch.Generator().manual_seed(1))
    assert total == 3 + 1 + 1 + 2 and table.shape == (4, 3)
    used = table[table >= 0]
    assert sorted(used.tolist()) == list(range(total))
    assert (table[1, 1:] == -1).all() and (table[2, 1:] == -1).all() and table[3, 2] == -1


def test_cache_rows_of_new_tokens():
    _, table = paged.gen_block_table([130, 7], 128, generator=torch.Generator().manual_seed(2))
    rows = paged.cache_rows_of_new_tokens([130, 7], table, 128, 2)
    assert rows[0].tolist() == [int(table[0, 1]) * 128 + 0, int(table[0, 1]) * 128 + 1]
    assert rows[1].tolist() == [int(table[1, 0]) * 128 + 5, int(table[1, 0]) * 128 + 6]


def test_topk_docstring_example():
    # python/pypto/op/comparison.py:333-341
    v, i = topk_rows(torch.tensor([[1.0, 2.0, 3.0], [1.0, 2.0, 3.0]]), 2)
    assert v.tolist() == [[3.0, 2.0], [3.0, 2.0]] and i.tolist() == [[2, 1], [2, 1]]


def test_topk_ties_take_smaller_index_first():
    # framework/src/interface/interpreter/calculator/calc_torch.cpp:2481-2494
    x = torch.tensor([5.0, 7.0, 5.0, 7.0, 1.0, 5.0])
    v, i = topk_sorted_stable(x, 5)
    assert i.tolist() == [1, 3, 0, 2, 5] and v.tolist() == [7.0, 7.0, 5.0, 5.0, 5.0]
    v, i = topk_sorted_stable(x, 3, largest=False)
    assert i.tolist() == [4, 0, 2]


@pytest.mark.parametrize("shape,k", [((64, 64), 10), ((4, 1000), 37), ((2, 4096), 2048)])
def test_topk_matches_torch_topk_values(shape, k):
    # framework/tests/st/operation/python/vector_operator_golden.py:2247-2259 defines top-k as torch.topk(sorted=True)
    x = torch.randn(shape, generator=torch.Generator().manual_seed(5))
    v, i = topk_rows(x, k)
    tv, _ = torch.topk(x, k, dim=-1, largest=True, sorted=True)
    assert torch.equal(v, tv)
    assert torch.equal(torch.gather(x, 1, i.long()), v)


def test_compare_threshold_and_rejections():
    ref = torch.ones(1000)
    t = ref.clone()
    t[:5] += 1.0  # 5 bad elements, limit round(0.005 * 1000) = 5
    assert compare(t, ref, "x", atol=1e-4, rtol=5e-3) == 5
    t[5] += 1.0
    with pytest.raises(AssertionError):
        compare(t, ref, "x", atol=1e-4, rtol=5e-3)
    bad = ref.clone()
    bad[0] = float("nan")
    with pytest.raises(AssertionError):
        compare(bad, ref, "x", 1.0, 1.0)
    bad[0] = float("inf")
    with pytest.raises(AssertionError):
        compare(bad, ref, "x", 1.0, 1.0)
    with pytest.raises(AssertionError):
        compare(ref[:10], ref, "x", 1.0, 1.0)
    with pytest.raises(AssertionError):
        compare(ref.double(), ref, "x", 1.0, 1.0)


def test_topk_idx_compare_is_set_based_per_group():
    ref = torch.arange(4096, dtype=torch.int32)
    perm = ref.clone()
    perm[:2048] = ref[:2048].flip(0)  # same ids inside the group, other positions
    assert topk_idx_compare(perm, ref, "ids") == 0
    one = ref.clone()
    one[7] = 99999
    assert topk_idx_compare(one, ref, "ids") == 1  # int(2048 * 5e-4) = 1 id may be missing
    two = one.clone()
    two[9] = 88888
    with pytest.raises(AssertionError):
        topk_idx_compare(two, ref, "ids")
    cross = ref.clone()  # ids moved to the other group count as missing there
    cross[0], cross[2048] = ref[2048], ref[0]
    cross[1], cross[2049] = ref[2049], ref[1]
    with pytest.raises(AssertionError):
        topk_idx_compare(cross, ref, "ids")
