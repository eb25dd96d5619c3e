"""The allocation-free entry point of sparse flash attention against the ordinary one.

pto_sfa_quant_launch_noalloc takes no workspace: the partial results of the KV splits go to an array that lives in the
library (one per GPU, held until the process ends).  Its output must equal pto_sfa_quant_launch's bit for bit - the same
kernels run on the same split - on two calls in a row, the second on a smaller problem (the array keeps what the
first call left in it).
"""
import ctypes

import pytest
import torch

from oracle import sfa as osfa
from oracle.compare import count_violations

from _cases import sfa_golden

pytestmark = pytest.mark.gpu


def both_entries(case, dev):
    from pypto_amd import _runtime
    lib = _runtime.load_library()
    fn = lib.pto_sfa_quant_launch_noalloc
    fn.restype = ctypes.c_int
    fn.argtypes = [ctypes.POINTER(_runtime.TensorDesc), ctypes.c_uint32, ctypes.POINTER(_runtime.SfaParams),
                   ctypes.c_void_p, ctypes.c_int]
    b, s1, nq, topk = case["b"], case["s1"], case["nq"], case["topk"]
    q = case["q"]
    ts = [q[..., :512].reshape(-1, 512).contiguous().to(dev), q[..., 512:].reshape(-1, 64).contiguous().to(dev),
          case["kn"].to(dev), case["kr"].to(dev), case["kn_scales"].to(dev), case["topk_indices"].to(dev),
          case["block_table"].to(dev), torch.tensor(case["act_seq"], dtype=torch.int32, device=dev)]
    p = _runtime.SfaParams(nq, 1, case["softmax_scale"], topk, case["block_size"], case["block_table"].shape[1], 0)
    stream = torch.cuda.current_stream().cuda_stream
    outs = []
    for static in (False, True):
        out = torch.full((b, s1, nq, 512), 7.0, dtype=torch.bfloat16, device=dev)
        d = _runtime.describe(ts + [out])
        if static:
            rc = fn(d, 9, ctypes.byref(p), stream, 1)
        else:
            n = lib.pto_sfa_quant_workspace(d, 9, ctypes.byref(p))
            assert n > 0, "the case must need scratch, or the test shows nothing"
            ws = torch.empty(n, dtype=torch.uint8, device=dev)
            rc = lib.pto_sfa_quant_launch(d, 9, ctypes.byref(p), ws.data_ptr(), n, stream, 1)
        assert rc == 0, lib.pto_last_error().decode()
        outs.append(out.cpu())
    return outs


def test_no_alloc_entry_matches_the_workspace_entry_twice(cuda):
    big = osfa.make_case(4, 128, 1, [5000, 900, 2048, 70], topk=2048, seed=71, dist="bench", softmax_scale=192 ** -0.5)
    small = osfa.make_case(2, 64, 2, [700, 300], topk=512, seed=72, dist="bench", softmax_scale=192 ** -0.5)
    for case in (big, small):
        want, got = both_entries(case, cuda)
        assert torch.isfinite(got.float()).all()
        assert torch.equal(got, want)
        # and on its own against the oracle, to the attention tests' bar (every element within 1e-2 + 2e-2 |golden|)
        assert count_violations(got, sfa_golden(case), 1e-2, 2e-2) == 0


def test_no_alloc_entry_rejects_what_does_not_fit(cuda):
    from pypto_amd import _runtime
    lib = _runtime.load_library()
    fn = lib.pto_sfa_quant_launch_noalloc
    fn.restype = ctypes.c_int
    fn.argtypes = [ctypes.POINTER(_runtime.TensorDesc), ctypes.c_uint32, ctypes.POINTER(_runtime.SfaParams),
                   ctypes.c_void_p, ctypes.c_int]
    # 64 query tokens x 16 forced splits x 128 heads need 135 MB of scratch; the array holds 40 MiB
    t, nq = 64, 128
    dev = cuda
    ts = [torch.zeros((t * nq, 512), dtype=torch.bfloat16, device=dev), torch.zeros((t * nq, 64), dtype=torch.bfloat16, device=dev),
          torch.zeros((256, 512), dtype=torch.int8, device=dev), torch.zeros((256, 64), dtype=torch.bfloat16, device=dev),
          torch.ones((256, 4), dtype=torch.float32, device=dev), torch.zeros((t, 2048), dtype=torch.int32, device=dev),
          torch.zeros((t, 2), dtype=torch.int32, device=dev), torch.full((t,), 100, dtype=torch.int32, device=dev),
          torch.zeros((t, 1, nq, 512), dtype=torch.bfloat16, device=dev)]
    p = _runtime.SfaParams(nq, 1, 0.1, 2048, 128, 2, 16)
    rc = fn(_runtime.describe(ts), 9, ctypes.byref(p), torch.cuda.current_stream().cuda_stream, 1)
    assert rc == -5 and b"scratch" in lib.pto_last_error()
