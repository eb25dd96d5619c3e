"""GPU parity: the standalone top-k operator (HIP, through the C ABI) against the CPU oracle.

Bar: values and indices bit-exact with the reference's golden, torch.topk(sorted=True)
(framework/tests/st/operation/python/vector_operator_golden.py:2247-2259), under the order its interpreter fixes for
equal values - smaller index first (framework/src/interface/interpreter/calculator/calc_torch.cpp:2481-2494).
"""
import pytest
import torch

from oracle import topk as otopk

pytestmark = pytest.mark.gpu

# the shape / k / largest columns of framework/tests/st/operation/test_case/TopK_st_test_cases.csv (values U[-100, 100])
ST_CASES = [((16, 128), -1, 10, False), ((32, 128), -1, 10, True), ((16, 128), 1, 10, False), ((32, 128), 1, 10, True),
            ((8, 8, 128), -1, 10, False), ((8, 8, 128), -1, 10, True), ((2, 8, 8, 128), -1, 10, False),
            ((2, 8, 8, 128), -1, 10, True), ((209, 40), -1, 40, False), ((739, 4257), -1, 4006, False)]


def check(x, k, dim, largest, dev):
    from pypto_amd.op import topk
    vals, idx = topk(x.to(dev), k, dim, largest)
    torch.cuda.synchronize()
    d = -1 if dim is None else dim
    x2 = x.movedim(d, -1)
    gv, gi = otopk.topk_rows(x2.reshape(-1, x2.shape[-1]), k, largest)
    gv = gv.reshape(*x2.shape[:-1], k).movedim(-1, d)
    gi = gi.reshape(*x2.shape[:-1], k).movedim(-1, d)
    assert vals.dtype == torch.float32 and idx.dtype == torch.int32 and vals.shape == gv.shape
    assert torch.equal(idx.cpu(), gi)
    assert torch.equal(vals.cpu().view(torch.int32), gv.view(torch.int32))  # bit for bit, the sign of zero included


def test_docstring_example(cuda):
    from pypto_amd.op import topk
    x = torch.tensor([[1.0, 2.0, 3.0], [1.0, 2.0, 3.0]])
    vals, idx = topk(x.to(cuda), 2, -1, True)
    assert vals.cpu().tolist() == [[3.0, 2.0], [3.0, 2.0]] and idx.cpu().tolist() == [[2, 1], [2, 1]]


@pytest.mark.parametrize("shape,dim,k,largest", ST_CASES)
def test_st_table_shapes(cuda, shape, dim, k, largest):
    g = torch.Generator().manual_seed(len(shape) * 1000 + k + largest)
    x = torch.rand(shape, generator=g) * 200 - 100
    check(x, k, dim, largest, cuda)


def test_ties_zero_signs_and_whole_rows(cuda):
    g = torch.Generator().manual_seed(5)
    x = torch.randint(-3, 4, (7, 300), generator=g).float()      # many exact ties
    x[0, ::3] = -0.0
    x[0, 1::3] = 0.0
    for largest in (True, False):
        check(x, 50, None, largest, cuda)
        check(x, 300, None, largest, cuda)                        # k = row length: a full stable sort
    check(torch.full((2, 1), 4.0), 1, None, True, cuda)
    check(torch.rand((3, 5, 9), generator=g), 4, 1, True, cuda)    # a middle dimension
    check(torch.rand((6, 17), generator=g), 3, 0, False, cuda)     # the first dimension


def test_row_slices_that_start_off_a_16_byte_boundary(cuda):
    # x[1:] of rows of 3 floats starts 12 bytes into the allocation and is contiguous: a legal operand as it is
    from pypto_amd.op import topk
    g = torch.Generator().manual_seed(9)
    x = torch.rand((5, 3), generator=g)
    xd = x.to(cuda)
    view = xd[1:]
    assert view.is_contiguous() and view.data_ptr() % 16 != 0
    vals, idx = topk(view, 2)
    gv, gi = otopk.topk_rows(x[1:], 2, True)
    assert torch.equal(idx.cpu(), gi) and torch.equal(vals.cpu(), gv)


def test_long_rows_go_through_the_radix_select(cuda):
    g = torch.Generator().manual_seed(6)
    x = torch.randn((3, 131072), generator=g)
    check(x, 2048, None, True, cuda)
    x = torch.randint(-50, 50, (2, 20000), generator=g).float()   # heavy ties across the selection boundary
    check(x, 1000, None, True, cuda)
    check(x, 17, None, False, cuda)


def test_errors(cuda):
    from pypto_amd.error import FeError
    from pypto_amd.op import topk
    x = torch.zeros((2, 10000), device=cuda)
    with pytest.raises(FeError, match="k <= 2048"):
        topk(x, 3000)
    with pytest.raises(FeError, match="1 <= k"):
        topk(x[:, :8].contiguous(), 9)
    with pytest.raises(FeError, match="float32"):
        topk(x.half(), 2)
