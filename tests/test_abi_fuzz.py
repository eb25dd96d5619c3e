"""No-GPU robustness of the boundary's validation: thousands of malformed calls of every ``pto_<op>_workspace`` entry
(which runs the operator's whole operand validation and launches nothing) must come back with a size or an error - no
crash, no division by zero, no absurd size.  Two generators: descriptor lists drawn at random (wrong counts, ranks,
dtypes, null and misaligned addresses, dimensions from 0 to 2^62 and negative), and valid lists with one to three
fields changed, which get past the first checks and reach the arithmetic behind them."""
import ctypes
import random

import pytest

from pypto_amd import _runtime as rt
from test_abi_host import BF16, FP32, INT8, INT32, apq_specs, descs, idx_specs, sfa_specs

OPS = {"sfa_quant": (rt.SfaParams, 9), "sfa_antiquant": (rt.SfaParams, 7), "lightning_indexer": (rt.IndexerParams, 8),
       "select_experts": (rt.SelectExpertsParams, 4), "gqa_decode": (rt.GqaParams, 6),
       "indexer_prolog": (rt.IndexerPrologParams, 21), "mla_prolog_quant": (rt.MlaPrologParams, 21),
       "mla_indexer_prolog_quant": (rt.MlaIndexerPrologParams, 34), "attention_pre_quant": (rt.AttentionPreQuantParams, 19),
       "paged_gather": (rt.PagedGatherParams, 4), "topk": (rt.TopkParams, 3)}
DIMS = [0, 1, 2, 3, 4, 7, 8, 16, 31, 32, 33, 64, 127, 128, 129, 192, 256, 512, 576, 640, 656, 1024, 1536, 2048, 2112, 4096,
        7168, 24576, 65536, 2 ** 31 - 1, 2 ** 31, 2 ** 40, 2 ** 62, -1, -128, -2 ** 31]
INTS = [0, 1, 2, 4, 8, 16, 64, 128, 2048, 4096, -1, 2 ** 31 - 1, -2 ** 31]
FLOATS = [0.0, 1.0, -1.0, 1e-6, 1e30, float("nan"), float("inf")]


@pytest.fixture(scope="module")
def lib():
    return rt.load_library()


def query(lib, op, arr, n, p):
    fn = getattr(lib, f"pto_{op}_workspace")
    fn.restype = ctypes.c_uint64
    size = fn(arr, n, p)
    assert size < 2 ** 48, f"{op}: workspace of {size} bytes"
    assert isinstance(lib.pto_last_error(), bytes)
    return size


def scramble_params(rng, p):
    for name, ty in p._fields_:
        setattr(p, name, rng.choice(FLOATS) if ty is ctypes.c_float else rng.choice(INTS))


def test_random_descriptor_lists(lib):
    rng = random.Random(1)
    for _ in range(600):
        for op, (params_type, n_tensors) in OPS.items():
            n = n_tensors if rng.random() < 0.8 else rng.choice([0, 1, n_tensors - 1, n_tensors + 1])
            arr = (rt.TensorDesc * max(n, 1))()
            for d in arr:
                d.addr = rng.choice([0, 0x1000, 0x1004, 0x1001, 0x7f0000001000])
                d.dataType = rng.choice([1, 3, 4, 6, 7, 8, 0, 2, 5, 9, 100, -1])
                d.rank = rng.choice([0, 1, 2, 2, 3, 3, 4, 4, 5, 8, 9, -1])
                for i in range(8):
                    d.shape[i] = rng.choice(DIMS)
            p = params_type()
            if rng.random() < 0.3:
                raw = (ctypes.c_ubyte * ctypes.sizeof(p)).from_buffer(p)
                for i in range(len(raw)):
                    raw[i] = rng.randrange(256)
            else:
                scramble_params(rng, p)
            query(lib, op, arr if n else None, n, ctypes.byref(p) if rng.random() < 0.97 else None)


def test_valid_lists_with_a_few_fields_changed(lib):
    templates = {
        "sfa_quant": (sfa_specs(), rt.SfaParams(128, 1, 0.1, 2048, 128, 8, 4)),
        "sfa_antiquant": ([(BF16, (256, 512)), (BF16, (256, 64)), (INT8, (1024, 656)), (INT32, (2, 2048)), (INT32, (2, 8)),
                           (INT32, (2,)), (BF16, (256, 512))], rt.SfaParams(128, 1, 0.1, 2048, 128, 8, 1)),
        "lightning_indexer": (idx_specs(), rt.IndexerParams(2048)),
        "topk": ([(FP32, (4, 100)), (FP32, (4, 10)), (INT32, (4, 10))], rt.TopkParams(10, 1)),
        "paged_gather": ([(INT8, (1024, 656)), (INT32, (2, 16)), (INT32, (2, 4)), (INT8, (32, 656))], rt.PagedGatherParams(128, 0)),
        "attention_pre_quant": (apq_specs(), rt.AttentionPreQuantParams(1e-5)),
    }
    rng = random.Random(2)
    for op, (specs, params) in templates.items():
        n = len(specs)
        assert query(lib, op, descs(specs), n, ctypes.byref(params)) >= 0   # the template itself is accepted
        for _ in range(2500):
            arr = descs(specs)
            p = type(params).from_buffer_copy(bytes(params))
            for _ in range(rng.choice([1, 1, 2, 3])):
                d = arr[rng.randrange(n)]
                what = rng.random()
                if what < 0.6:
                    d.shape[rng.randrange(8)] = rng.choice(DIMS)
                elif what < 0.75:
                    d.rank = rng.choice([0, 1, 2, 3, 4, 5, 8, 9, -1])
                elif what < 0.9:
                    d.dataType = rng.choice([1, 3, 4, 6, 7, 8, 0, 2, 100, -1])
                else:
                    d.addr = rng.choice([0, 0x1000, 0x1004, 0x1001])
            if rng.random() < 0.4:
                name, ty = rng.choice(p._fields_)
                setattr(p, name, rng.choice(FLOATS) if ty is ctypes.c_float else rng.choice(INTS))
            query(lib, op, arr, n, ctypes.byref(p))
