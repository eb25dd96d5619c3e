"""Host logic of the operator boundary: the plan a call leaves for the next call of the same operator (CPU only; the
C entry points are replaced by recorders)."""
import ctypes

import pytest
import torch

from pypto_amd import _runtime as rt


@pytest.fixture
def recorder(monkeypatch):
    calls = []

    def ws_fn(descs, n, p):
        calls.append(("workspace", n))
        return 0

    def launch_fn(descs, n, p, ws, ws_bytes, stream, sync):
        calls.append(("launch", [descs[i].addr for i in range(n)],
                      [tuple(descs[i].shape[:descs[i].rank]) for i in range(n)],
                      ctypes.cast(p, ctypes.POINTER(rt.TopkParams)).contents.k))
        return 0

    def describe_with_buf(tensors):
        n = len(tensors)
        buf = bytearray(rt._DESC.size * n)
        off = 0
        for t in tensors:
            shape = t.shape
            rt._DESC.pack_into(buf, off, t.data_ptr() if t.numel() else 0, rt._DTYPE_CODE[t.dtype], len(shape), *shape,
                               *rt._PAD[len(shape)])
            off += rt._DESC.size
        d = (rt.TensorDesc * n).from_buffer(buf)
        d._buf = buf
        return d

    def check2(tensors):
        for t in tensors:
            if not t.is_contiguous():
                raise rt.FeError(RuntimeError("not all tensors are contiguous"))
        return tensors[0].device, describe_with_buf(tensors)

    monkeypatch.setattr(rt, "_check_and_describe", check2)
    monkeypatch.setattr(rt, "_entry_points", lambda op: (ws_fn, launch_fn))
    monkeypatch.setattr(rt, "_launch_on_current_device",
                        lambda dev, fn, descs, n, pref, wsb: fn(descs, n, pref, None, wsb, None, 0))
    rt._tls.plans = {}
    return calls


def test_repeated_call_skips_validation_and_workspace_query(recorder):
    x, v, i = torch.zeros(4, 100), torch.zeros(4, 10), torch.zeros(4, 10, dtype=torch.int32)
    p = rt.TopkParams(10, 1)
    rt.launch("topk", [x, v, i], p)
    rt.launch("topk", [x, v, i], p)
    assert [c[0] for c in recorder] == ["workspace", "launch", "launch"]
    assert recorder[1][1:] == recorder[2][1:] and recorder[2][1][0] == x.data_ptr()


def test_new_storage_under_the_same_tensor_is_picked_up(recorder):
    x, v, i = torch.zeros(4, 100), torch.zeros(4, 10), torch.zeros(4, 10, dtype=torch.int32)
    p = rt.TopkParams(10, 1)
    rt.launch("topk", [x, v, i], p)
    old = x.data_ptr()
    x.set_(torch.ones(4, 100))  # same object, same shape, another allocation
    assert x.data_ptr() != old
    rt.launch("topk", [x, v, i], p)
    assert [c[0] for c in recorder] == ["workspace", "launch", "launch"]
    assert recorder[2][1][0] == x.data_ptr()


def test_operands_that_change_are_described_afresh(recorder):
    x, v, i = torch.zeros(4, 100), torch.zeros(4, 10), torch.zeros(4, 10, dtype=torch.int32)
    rt.launch("topk", [x, v, i], rt.TopkParams(10, 1))
    x2 = x.clone()
    rt.launch("topk", [x2, v, i], rt.TopkParams(10, 1))               # another object of the same shape: no new sizing
    assert [c[0] for c in recorder] == ["workspace", "launch", "launch"] and recorder[2][1][0] == x2.data_ptr()
    rt.launch("topk", [x, v, i], rt.TopkParams(10, 0))                # other scalar parameters: sized again
    x.resize_(4, 50)
    rt.launch("topk", [x, v, i], rt.TopkParams(10, 0))                # the same object with another shape: sized again
    assert [c[0] for c in recorder] == ["workspace", "launch", "launch", "workspace", "launch", "workspace", "launch"]
    assert recorder[-1][2][0] == (4, 50) and recorder[4][3] == 10
    with pytest.raises(rt.FeError, match="same device"):
        rt.launch("topk", [x, v, torch.zeros(4, 10, dtype=torch.int32, device="meta")], rt.TopkParams(10, 0))
    y = torch.zeros(6, 4).t()
    with pytest.raises(rt.FeError, match="contiguous"):
        rt.launch("topk", [y, v, i], rt.TopkParams(10, 0))
    x2 = torch.zeros(4, 100)
    rt.launch("topk", [x2, v, i], rt.TopkParams(10, 1))
    x2.t_()                                                            # the same object, no longer dense
    with pytest.raises(rt.FeError, match="contiguous"):
        rt.launch("topk", [x2, v, i], rt.TopkParams(10, 1))


def test_a_dead_tensor_never_matches(recorder):
    v, i = torch.zeros(4, 10), torch.zeros(4, 10, dtype=torch.int32)
    p = rt.TopkParams(10, 1)
    ptrs = []
    for _ in range(3):
        x = torch.zeros(4, 100)                                      # a fresh input every call
        ptrs.append(x.data_ptr())
        rt.launch("topk", [x, v, i], p)
    assert [c[0] for c in recorder] == ["workspace", "launch", "launch", "launch"]
    assert [c[1][0] for c in recorder if c[0] == "launch"] == ptrs
