"""Host logic of the operator boundary: the pybind11 layer's operand checks and descriptor list (CPU only: describe() is
the validation half of launch(); the launch itself needs a HIP device and is what every GPU test goes through)."""
import ctypes

import pytest
import torch

from pypto_amd import _runtime as rt
from pypto_amd.error import FeError


@pytest.fixture(scope="module")
def host():
    return rt.load_host()


def unpack(blob):
    n = len(blob) // ctypes.sizeof(rt.TensorDesc)
    arr = (rt.TensorDesc * n).from_buffer_copy(blob)
    return [(d.addr or 0, d.dataType, tuple(d.shape[:d.rank])) for d in arr]


def test_descriptor_list_matches_the_ctypes_binding(host):
    ts = [torch.zeros(4, 100), torch.zeros(4, 10, dtype=torch.bfloat16), torch.zeros(4, 10, dtype=torch.int32),
          torch.zeros(2, 3, 4, 5, dtype=torch.int8), torch.zeros(7, dtype=torch.float16), torch.zeros(3, dtype=torch.int64),
          torch.zeros(0, 5)]
    blob, dev = host.describe(ts)
    assert dev == "cpu"
    assert blob == bytes(rt.describe(ts))
    got = unpack(blob)
    assert [g[1] for g in got] == [7, 8, 3, 1, 6, 4, 7]
    assert got[0] == (ts[0].data_ptr(), 7, (4, 100)) and got[3][2] == (2, 3, 4, 5)
    assert got[6][0] == 0                                            # an empty tensor carries a null address
    assert host.describe(tuple(ts))[0] == blob                       # any sequence


def test_every_call_describes_the_operands_as_they_are_now(host):
    # a Parameter moved by .data = (what nn.Module.to() / .half() do): same object, other dtype and storage
    x = torch.zeros(4, 100)
    before = unpack(host.describe([x])[0])[0]
    x.data = x.data.to(torch.bfloat16)
    after = unpack(host.describe([x])[0])[0]
    assert before[1] == 7 and after[1] == 8 and after[0] == x.data_ptr()
    x.set_(torch.ones(4, 50, dtype=torch.bfloat16))                  # same object, another allocation and shape
    assert unpack(host.describe([x])[0])[0] == (x.data_ptr(), 8, (4, 50))
    # operands on one device, then all on another: nothing is remembered between calls
    assert host.describe([torch.zeros(3), torch.zeros(3)])[1] == "cpu"
    assert host.describe([torch.zeros(3, device="meta"), torch.zeros(3, device="meta")])[1] == "meta"
    assert host.describe([torch.zeros(3), torch.zeros(3)])[1] == "cpu"


def test_operand_checks_of_the_reference_binding(host):
    x = torch.zeros(4, 100)
    with pytest.raises(host.BindingError, match=r"Input 2 \(index 1\) must be a torch.Tensor"):
        host.describe([x, 3])
    with pytest.raises(host.BindingError, match="contiguous"):
        host.describe([x, torch.zeros(6, 4).t()])
    with pytest.raises(host.BindingError, match="same device, got cpu and meta"):
        host.describe([x, torch.zeros(3, device="meta")])
    with pytest.raises(ValueError, match="unsupported tensor dtype"):
        host.describe([x, torch.zeros(3, dtype=torch.float64)])
    with pytest.raises(ValueError, match="8 dimensions"):
        host.describe([torch.zeros((1,) * 9)])

    class DTensor(torch.Tensor):                                     # (the reference rejects the type by its name)
        pass

    with pytest.raises(host.BindingError, match="must not be a DTensor"):
        host.describe([x, torch.zeros(3).as_subclass(DTensor)])

    class Plain(torch.Tensor):
        pass

    assert unpack(host.describe([torch.zeros(3).as_subclass(Plain)])[0])[0][2] == (3,)
    x2 = torch.zeros(4, 100)
    x2.t_()                                                          # a dense tensor made non-dense in place
    with pytest.raises(host.BindingError, match="contiguous"):
        host.describe([x2])


def test_launch_rejects_before_any_c_call(host):
    x, v, i = torch.zeros(4, 100), torch.zeros(4, 10), torch.zeros(4, 10, dtype=torch.int32)
    with pytest.raises(FeError, match="HIP device"):                 # binding-level failures surface as FeError as they are
        rt.launch("topk", [x, v, i], rt.TopkParams(10, 1))
    with pytest.raises(FeError, match="contiguous"):
        rt.launch("topk", [torch.zeros(100, 4).t(), v, i], rt.TopkParams(10, 1))
    with pytest.raises(ValueError, match="parameter block of 4 bytes, expected 8"):
        host.launch(host.OPS["topk"], [x, v, i], bytes(4))
    with pytest.raises(ValueError, match="unknown operator id"):
        host.launch(99, [x, v, i], bytes(8))
    with pytest.raises(FeError, match="no tensors"):
        rt.launch("topk", [], rt.TopkParams(10, 1))


def test_parameter_blocks_agree_with_the_header(host):
    assert set(host.OPS) == set(rt._OPS)
    for op, ptype in rt._OPS.items():
        assert host.PARAM_BYTES[op] == ctypes.sizeof(ptype), op
    assert host.ABI_VERSION == rt.ABI_VERSION == rt.load_library().pto_abi_version()
