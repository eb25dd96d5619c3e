"""GPU parity: paged row gather (HIP, through the C ABI) against the CPU oracle.  Bar: bit-exact for every dtype."""
import pytest
import torch

from oracle import paged

pytestmark = pytest.mark.gpu

DTYPES = (torch.int8, torch.float16, torch.bfloat16, torch.float32, torch.int32, torch.int64)


def make_src(n, hidden, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    if dtype.is_floating_point:
        return torch.randn((n, hidden), generator=g).to(dtype)
    hi = 127 if dtype == torch.int8 else 1 << 30
    return torch.randint(-hi, hi + 1, (n, hidden), generator=g, dtype=torch.int64).to(dtype)


def bits(t):
    return t.contiguous().view(torch.uint8)


def test_reference_docstring_example(cuda):
    # python/pypto/experimental/gather.py:57-82
    from pypto_amd.experimental import gather_in_ub
    src = torch.arange(24, dtype=torch.float32).reshape(6, 4)
    idx = torch.tensor([[0, 4, 3]], dtype=torch.int32)
    page = torch.tensor([[0, 2, 1]], dtype=torch.int32)
    out = gather_in_ub(src.to(cuda), idx.to(cuda), page.to(cuda), 2, -2, check=True).cpu()
    assert out.tolist() == [[0, 1, 2, 3], [8, 9, 10, 11], [20, 21, 22, 23]]


def test_reference_st_case(cuda):
    # python/tests/st/operation/vector/test_gatherinub.py:83-130,205-229: buffer[tok, h] = 10*tok + h (fp16, 32 x 4),
    # block size 4, a shuffled page table and 8 logical indices
    from pypto_amd.experimental import gather_in_ub
    buf = (10 * torch.arange(32).reshape(32, 1) + torch.arange(4).reshape(1, 4)).to(torch.float16)
    page = torch.tensor([[3, 0, 7, 1, 5, 2, 6, 4]], dtype=torch.int32)
    idx = torch.tensor([[0, 5, 9, 14, 18, 23, 27, 31]], dtype=torch.int32)
    out = gather_in_ub(buf.to(cuda), idx.to(cuda), page.to(cuda), 4, -2, check=True).cpu()
    for j, i in enumerate(idx[0].tolist()):
        tok = int(page[0, i // 4]) * 4 + i % 4
        assert out[j].tolist() == [10 * tok + h for h in range(4)]
    assert torch.equal(out, paged.paged_gather(buf, idx[0], page[0], 4))


@pytest.mark.parametrize("dtype", DTYPES)
def test_dtypes_and_widths_bit_exact(cuda, dtype):
    from pypto_amd.experimental import gather_in_l1, gather_in_ub
    # widths that take the 16-, 8-, 4-, 2- and 1-byte copy paths for the dtype's element size
    for seed, (hidden, size, bs, nblk, k) in enumerate([(512, 512, 128, 9, 300), (656, 656, 16, 40, 77), (36, 20, 4, 13, 33),
                                                        (7, 7, 3, 5, 15), (129, 1, 8, 6, 41), (64, 63, 2, 50, 100)]):
        n = nblk * bs
        src = make_src(n, hidden, dtype, 100 + seed)
        g = torch.Generator().manual_seed(seed)
        page = torch.randperm(nblk, generator=g).to(torch.int32).reshape(1, nblk)
        idx = torch.randint(0, n, (1, k), generator=g, dtype=torch.int32)
        want = paged.paged_gather(src, idx[0], page[0], bs)[:, :size]
        if size == hidden:
            got = gather_in_ub(src.to(cuda), idx.to(cuda), page.to(cuda), bs, -2, check=True)
        else:
            got = gather_in_l1(src.to(cuda), idx.to(cuda), page.to(cuda), bs, size, check=True)
        assert got.shape == want.shape and got.dtype == dtype
        assert torch.equal(bits(got.cpu()), bits(want)), (dtype, hidden, size)


def test_batched_rows_and_index_dtypes(cuda):
    from pypto_amd.experimental import paged_gather
    b, bs, k, hidden = 5, 128, 2048, 656  # the packed 656-byte cache row of the antiquant attention entry
    act = [4000, 129, 128, 9000, 2048]
    g = torch.Generator().manual_seed(7)
    total, table = paged.gen_block_table(act, bs, generator=g)
    src = make_src(total * bs, hidden, torch.int8, 3)
    idx = torch.stack([torch.randint(0, a, (k,), generator=g) for a in act])
    want = torch.cat([paged.paged_gather(src, idx[i], table[i].clamp_min(0), bs) for i in range(b)])
    for idt in (torch.int32, torch.int64):
        for bdt in (torch.int32, torch.int64):
            got = paged_gather(src.to(cuda), idx.to(idt).to(cuda), table.to(bdt).to(cuda), bs, check=True)
            assert torch.equal(got.cpu(), want), (idt, bdt)


def test_unaligned_views_take_the_narrow_paths(cuda):
    # a source whose base address is only 2-byte aligned and whose pitch is odd in 16-byte units
    from pypto_amd._runtime import PagedGatherParams, launch
    bs, nblk, k = 4, 8, 19
    n = bs * nblk
    flat = make_src(1, n * 24 + 8, torch.bfloat16, 5).reshape(-1).to(cuda)
    src = flat[1:1 + n * 24].view(n, 24)
    g = torch.Generator().manual_seed(11)
    page = torch.randperm(nblk, generator=g).to(torch.int32).reshape(1, nblk)
    idx = torch.randint(0, n, (1, k), generator=g, dtype=torch.int32)
    out = torch.empty((k, 24), dtype=torch.bfloat16, device=cuda)
    launch("paged_gather", [src, idx.to(cuda), page.to(cuda), out], PagedGatherParams(bs, 24))
    want = paged.paged_gather(src.cpu(), idx[0], page[0], bs)
    assert torch.equal(bits(out.cpu()), bits(want))


def test_entries_the_interpreter_rejects(cuda):
    # framework/src/interface/interpreter/calculator/calc_torch.cpp:1916-1950 asserts on these; the kernel writes a zero
    # row for each and counts it, and check=True turns the count into the interpreter's error
    from pypto_amd.error import FeError
    from pypto_amd.experimental import paged_gather
    src = make_src(12, 8, torch.float32, 1)
    page = torch.tensor([[0, -1, 2, 9]], dtype=torch.int32)          # page 1 unused, page 3 beyond the 12 source rows
    idx = torch.tensor([[0, 5, 3, 9, 12, 16, -1, 13]], dtype=torch.int32)  # 16 and -1 lie outside the table
    got = paged_gather(src.to(cuda), idx.to(cuda), page.to(cuda), 4).cpu()
    good = {0: 0, 2: 3, 3: 9}
    for j in range(8):
        assert torch.equal(got[j], src[good[j]] if j in good else torch.zeros(8)), j
    with pytest.raises(FeError, match="5 of 8 indices"):
        paged_gather(src.to(cuda), idx.to(cuda), page.to(cuda), 4, check=True)
    for i in (16, -1):
        with pytest.raises(IndexError):
            paged.paged_gather(src, [i], page[0], 4)


def test_empty_and_argument_errors(cuda):
    from pypto_amd.error import FeError
    from pypto_amd.experimental import gather_in_l1, gather_in_ub, paged_gather
    src = make_src(8, 4, torch.float16, 0).to(cuda)
    page = torch.tensor([[0, 1]], dtype=torch.int32, device=cuda)
    idx = torch.zeros((1, 0), dtype=torch.int32, device=cuda)
    assert gather_in_ub(src, idx, page, 4, -2).shape == (0, 4)
    idx = torch.tensor([[1, 2]], dtype=torch.int32, device=cuda)
    assert gather_in_l1(src, idx, page, 4, 0).shape == (2, 0)
    with pytest.raises(FeError, match="axis"):
        gather_in_ub(src, idx, page, 4, -1)
    with pytest.raises(FeError, match="size"):
        gather_in_l1(src, idx, page, 4, 5)
    with pytest.raises(FeError, match="block_size"):
        paged_gather(src, idx, page, 0)
    with pytest.raises(FeError, match="int32 or int64"):
        paged_gather(src, idx.to(torch.int16), page, 4)
    with pytest.raises(FeError, match="rows"):
        paged_gather(src, idx.expand(2, 2).contiguous(), page, 4)


def test_gathered_rows_are_what_attention_reads(cuda):
    # the attention kernel resolves the same index -> page -> row chain internally: gathering the selected rows of
    # the three cache tensors first and attending over them as a dense, identity-paged cache gives the same output bits
    from oracle import sfa as osfa
    from pypto_amd.experimental import paged_gather
    from tests._cases import run_sfa
    b, k, bs = 2, 256, 128
    case = osfa.make_case(b, 16, 1, [700, 1300], topk=k, block_size=bs, seed=21, dist="bench")
    out_paged = run_sfa(case, cuda)
    idx, table = case["topk_indices"].to(cuda), case["block_table"].to(cuda)
    dense = dict(case)
    for name in ("kn", "kr", "kn_scales"):
        dense[name] = paged_gather(case[name].to(cuda), idx, table, bs, check=True).cpu()
        want = torch.cat([paged.paged_gather(case[name], case["topk_indices"][i], case["block_table"][i].clamp_min(0), bs)
                          for i in range(b)])
        assert torch.equal(bits(dense[name]), bits(want)), name
    dense["block_table"] = torch.arange(b * k // bs, dtype=torch.int32).reshape(b, k // bs)
    dense["topk_indices"] = torch.arange(k, dtype=torch.int32).reshape(1, k).expand(b, k).contiguous()
    dense["act_seq"] = [k, k]
    out_dense = run_sfa(dense, cuda)
    assert torch.equal(bits(out_paged), bits(out_dense))
