"""No-GPU checks of the boundary: the C-ABI library loads and exports every symbol include/pypto_amd.h declares,
its operand validation rejects bad calls with the documented codes (no compute call is made), and the Python
operator layer mirrors the reference's call convention and error wrapping."""
import ctypes
import os
import re

import pytest
import torch

from pypto_amd import _runtime
from pypto_amd._runtime import IndexerParams, SfaParams, TensorDesc
from pypto_amd.deepseek_v32_exp import lightning_indexer_quant_impl as li
from pypto_amd.deepseek_v32_exp import sparse_attention_antiquant_impl as aq
from pypto_amd.deepseek_v32_exp import sparse_flash_attention_quant_impl as sfa
from pypto_amd.error import FeError, PyptoError

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
INT8, INT32, FP16, FP32, BF16 = 1, 3, 6, 7, 8
FAKE = 0x1000  # never dereferenced: validation only


@pytest.fixture(scope="module")
def lib():
    return _runtime.load_library()


def descs(specs):
    arr = (TensorDesc * len(specs))()
    for d, (dt, shape) in zip(arr, specs):
        d.addr, d.dataType, d.rank = FAKE, dt, len(shape)
        for i, s in enumerate(shape):
            d.shape[i] = s
    return arr


def sfa_specs(t=2, nq=128, n=1024, topk=2048, b=2, blocks=8, kn_dt=INT8):
    return [(BF16, (t * nq, 512)), (BF16, (t * nq, 64)), (kn_dt, (n, 512)), (BF16, (n, 64)), (FP32, (n, 4)),
            (INT32, (t, topk)), (INT32, (b, blocks)), (INT32, (b,)), (BF16, (b, t // b, nq, 512))]


def idx_specs(t=2, b=2, blocks=16, bs=128, mb=8, k=2048):
    return [(INT8, (t, 64, 128)), (FP16, (t, 64)), (INT8, (blocks, bs, 1, 128)), (FP16, (blocks, bs, 1)),
            (FP16, (t, 64)), (INT32, (b,)), (INT32, (b, mb)), (INT32, (t, 1, k))]


def test_every_declared_symbol_is_exported(lib):
    header = open(os.path.join(ROOT, "include", "pypto_amd.h")).read()
    names = set(re.findall(r"\b(pto_[a-z_0-9]+)\s*\(", header))
    assert {"pto_sfa_quant_launch", "pto_sfa_antiquant_launch", "pto_lightning_indexer_launch",
            "pto_last_error"} <= names
    for n in names:
        assert hasattr(lib, n), f"{n} declared in the header but not exported"
    assert lib.pto_abi_version() == 2


def test_topk_validation_codes(lib):
    from pypto_amd._runtime import TopkParams
    ok = [(FP32, (4, 100)), (FP32, (4, 10)), (INT32, (4, 10))]
    p = TopkParams(10, 1)
    assert launch_rc(lib, "topk", ok[:2], p)[0] == -1
    assert launch_rc(lib, "topk", [(BF16, (4, 100))] + ok[1:], p)[0] == -2
    assert launch_rc(lib, "topk", [ok[0], (FP32, (4, 9)), ok[2]], p)[0] == -3
    rc, msg = launch_rc(lib, "topk", [(FP32, (4, 9000)), (FP32, (4, 3000)), (INT32, (4, 3000))], TopkParams(3000, 1))
    assert rc == -4 and "k <= 2048" in msg
    assert launch_rc(lib, "topk", [(FP32, (4, 5)), (FP32, (4, 6)), (INT32, (4, 6))], TopkParams(6, 0))[0] == -4


def test_tensor_desc_layout_matches_the_reference_abi():
    # framework/include/tile_fwk_bundle/pypto_bundle_api.h:30-35: void* | int32 | int32 | int64[8]
    assert ctypes.sizeof(TensorDesc) == 8 + 4 + 4 + 64
    assert TensorDesc.dataType.offset == 8 and TensorDesc.rank.offset == 12 and TensorDesc.shape.offset == 16
    assert _runtime._DTYPE_CODE == {torch.int8: 1, torch.int32: 3, torch.int64: 4, torch.float16: 6, torch.float32: 7,
                                    torch.bfloat16: 8}


def test_sfa_workspace_query(lib):
    p = SfaParams(128, 1, 0.1, 2048, 128, 8, 4)
    ws = lib.pto_sfa_quant_workspace(descs(sfa_specs()), 9, ctypes.byref(p))
    assert ws == 2 * 4 * 128 * (512 * 2 + 2 * 4)  # t * splits * nq * (512 fp16 + (m, l) fp32)
    p.kv_splits = 1
    assert lib.pto_sfa_quant_workspace(descs(sfa_specs()), 9, ctypes.byref(p)) == 0  # single pass: no scratch
    p.kv_splits = 0  # automatic: some positive split count on a 256-CU part, never more than 16
    auto = lib.pto_sfa_quant_workspace(descs(sfa_specs()), 9, ctypes.byref(p))
    assert auto % (2 * 128 * 1032) == 0 and 1 <= auto // (2 * 128 * 1032) <= 16


def launch_rc(lib, op, specs, params, ws=None, ws_bytes=0):
    fn = getattr(lib, f"pto_{op}_launch")
    rc = fn(descs(specs), len(specs), ctypes.byref(params), ws, ws_bytes, None, 0)
    return rc, lib.pto_last_error().decode()


def test_misaligned_addresses_are_refused(lib):
    """The kernels read and write 16 bytes per lane: an address that is not a multiple of 16 is refused with its own
    code (-8) before anything is launched; the paged gather asks only for element alignment."""
    from pypto_amd._runtime import PagedGatherParams
    p = SfaParams(128, 1, 0.1, 2048, 128, 8, 4)
    d = descs(sfa_specs())
    d[0].addr = FAKE + 8
    fn = lib.pto_sfa_quant_launch
    assert fn(d, 9, ctypes.byref(p), None, 0, None, 0) == -8
    assert "query_nope" in lib.pto_last_error().decode() and "16 bytes" in lib.pto_last_error().decode()
    assert lib.pto_sfa_quant_workspace(d, 9, ctypes.byref(p)) == 0
    # (the page table has one row too many, so that the call is refused after the address checks and launches nothing)
    g = descs([(BF16, (64, 24)), (INT32, (2, 8)), (INT32, (3, 4)), (BF16, (16, 24))])
    gp = PagedGatherParams(16, 0)
    g[0].addr, g[3].addr = FAKE + 2, FAKE + 6     # views that start inside a row: fine for the gather
    assert lib.pto_paged_gather_launch(g, 4, ctypes.byref(gp), None, 0, None, 0) == -3, lib.pto_last_error().decode()
    g[0].addr = FAKE + 1                          # not even an element boundary
    assert lib.pto_paged_gather_launch(g, 4, ctypes.byref(gp), None, 0, None, 0) == -8


def test_sfa_validation_codes(lib):
    p = SfaParams(128, 1, 0.1, 2048, 128, 8, 4)
    rc, msg = launch_rc(lib, "sfa_quant", sfa_specs()[:8], p)
    assert rc == -1 and "expected 9 tensors" in msg
    bad = sfa_specs(); bad[0] = (FP16, bad[0][1])
    rc, msg = launch_rc(lib, "sfa_quant", bad, p)
    assert rc == -2 and "query_nope must be bf16" in msg
    bad = sfa_specs(); bad[2] = (FP32, bad[2][1])
    assert launch_rc(lib, "sfa_quant", bad, p)[0] == -2  # cache must be int8 or bf16
    bad = sfa_specs(); bad[1] = (BF16, (256, 32))
    rc, msg = launch_rc(lib, "sfa_quant", bad, p)
    assert rc == -3 and "query_rope" in msg
    bad = sfa_specs(); bad[6] = (INT32, (2, 9))
    assert launch_rc(lib, "sfa_quant", bad, p)[0] == -3  # block_table width != max_blocknum_perbatch
    bad = sfa_specs(); bad[5] = (INT32, (2, 100))
    assert launch_rc(lib, "sfa_quant", bad, p)[0] == -3  # fewer index columns than topk
    for field, value in (("n_kv", 2), ("topk", 4096), ("topk", 0), ("block_size", 0), ("kv_splits", 99)):
        q = SfaParams(128, 1, 0.1, 2048, 128, 8, 4)
        setattr(q, field, value)
        assert launch_rc(lib, "sfa_quant", sfa_specs(), q)[0] == -4, field
    q = SfaParams(128, 1, float("nan"), 2048, 128, 8, 4)
    assert launch_rc(lib, "sfa_quant", sfa_specs(), q)[0] == -4
    rc, msg = launch_rc(lib, "sfa_quant", sfa_specs(), p)  # needs a workspace, none given
    assert rc == -5 and "workspace" in msg
    null = descs(sfa_specs()); null[3].addr = None
    assert lib.pto_sfa_quant_launch(null, 9, ctypes.byref(p), None, 0, None, 0) == -6
    assert lib.pto_sfa_quant_workspace(descs(sfa_specs()), 9, None) == 0  # query reports failure as 0


def test_antiquant_validation(lib):
    p = SfaParams(128, 1, 0.1, 2048, 128, 8, 1)
    specs = [(BF16, (256, 512)), (BF16, (256, 64)), (INT8, (1024, 656)), (INT32, (2, 2048)), (INT32, (2, 8)),
             (INT32, (2,)), (BF16, (256, 512))]
    assert lib.pto_sfa_antiquant_workspace(descs(specs), 7, ctypes.byref(p)) == 0
    bad = list(specs); bad[2] = (INT8, (1024, 640))
    rc, msg = launch_rc(lib, "sfa_antiquant", bad, p)
    assert rc == -3 and "656" in msg
    bad = list(specs); bad[6] = (BF16, (2, 1, 128, 512))
    assert launch_rc(lib, "sfa_antiquant", bad, p)[0] == -3  # this entry's output is 2-D
    assert launch_rc(lib, "sfa_antiquant", specs[:6], p)[0] == -1


def test_indexer_validation_and_workspace(lib):
    p = IndexerParams(2048)
    ws = lib.pto_lightning_indexer_workspace(descs(idx_specs()), 8, ctypes.byref(p))
    assert ws >= 2 * 8 * 128 * 4  # at least the dense score rows
    rc, msg = launch_rc(lib, "lightning_indexer", idx_specs(), p)
    assert rc == -5
    bad = idx_specs(); bad[0] = (INT8, (2, 32, 128))
    assert launch_rc(lib, "lightning_indexer", bad, p)[0] == -3  # 64 index heads of 128
    bad = idx_specs(); bad[1] = (FP32, (2, 64))
    assert launch_rc(lib, "lightning_indexer", bad, p)[0] == -2
    bad = idx_specs(t=10, b=2)
    assert launch_rc(lib, "lightning_indexer", bad, p)[0] == -3  # 5 query tokens per sequence > 4
    bad = idx_specs(); bad[7] = (INT32, (2, 1, 1024))
    assert launch_rc(lib, "lightning_indexer", bad, p)[0] == -3
    assert launch_rc(lib, "lightning_indexer", idx_specs(k=4096), IndexerParams(4096))[0] == -4
    assert launch_rc(lib, "lightning_indexer", idx_specs()[:7], p)[0] == -1


def test_operator_call_convention_and_error_wrapping():
    t = [torch.zeros(1)] * 9
    cfg = sfa.SaTileShapeConfig(g_tile=128, s_kv_tile=2048, gather_vec_tile_shape=[32, 512],
                                c1_tile_shape=[128] * 6, v1_tile_shape=[8, 2048], c2_tile_shape=[128] * 6,
                                v2_tile_shape=[64, 256])
    with pytest.raises(FeError) as e:  # CPU tensors: refused before any native call
        sfa.sparse_flash_attention_quant_d(*t, 128, 1, 0.1, 2048, 128, 8, cfg)
    assert "ErrCode" in str(e.value) and "RuntimeError" in str(e.value)
    with pytest.raises(FeError):  # non-tensor arguments may come by keyword
        sfa.sparse_flash_attention_quant_d(*t, 128, 1, softmax_scale=0.1, topk=2048, block_size=128,
                                           max_blocknum_perbatch=8, tile_config=cfg)
    with pytest.raises(FeError) as e:
        sfa.sparse_flash_attention_quant_d(*t, 128, 1, 0.1, 2048, 128, 8)  # tile_config missing
    assert "TypeError" in str(e.value) and "Failed to call JIT function 'sparse_flash_attention_quant_d'" in str(e.value)
    with pytest.raises(FeError):
        sfa.sparse_flash_attention_quant_d(*t, 128, 1, 0.1, 2048, 128, 8, cfg, bogus=1)
    with pytest.raises(FeError) as e:
        sfa.sparse_flash_attention_quant_d(*t[:8], "not a tensor", 128, 1, 0.1, 2048, 128, 8, cfg)
    assert "must be a torch.Tensor" in str(e.value)
    nc = torch.zeros((4, 4)).t()
    with pytest.raises(FeError) as e:
        sfa.sparse_flash_attention_quant_p(nc, *t[1:], 128, 1, 0.1, 2048, 128, 8, cfg)
    assert "contiguous" in str(e.value)
    with pytest.raises(FeError):
        aq.sparse_attention_antiquant_d(*t[:7], 128, 1, 0.1, 2048, 128, 8, aq.SaTileShapeConfig())
    with pytest.raises(FeError):
        li.lightning_indexer_decode(*t[:8], [128, 64], li.LightningIndexerConfigs(), 2048)
    assert issubclass(FeError, PyptoError)
    assert sfa.sparse_flash_attention_quant_d.__name__ == "sparse_flash_attention_quant_d"
    assert li.MAX_LI_S1 == 4 and li.MAX_LI_S2 == 128 * 1024


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    monkeypatch.setattr(_runtime, "_lib", None)
    monkeypatch.setattr(_runtime, "_LIB_PATH", str(tmp_path / "libpypto_amd.so"))
    with pytest.raises(PyptoError) as e:
        _runtime.load_library()
    assert "python -m pypto_amd.build" in str(e.value)


def apq_specs(t=8, h=5120, q=1536, kv=128, d=128, half=32):
    n_out = q + 2 * kv
    return [(BF16, (t, h)), (BF16, (t, h)), (BF16, (h,)), (BF16, (h,)), (BF16, (h,)), (BF16, (h,)), (INT8, (h, n_out)),
            (INT32, (n_out,)), (FP32, (n_out,)), (BF16, (d,)), (BF16, (d,)), (BF16, (d,)), (BF16, (d,)),
            (BF16, (t, 1, half)), (BF16, (t, 1, half)), (BF16, (t, q)), (BF16, (t, kv)), (BF16, (t, kv)), (BF16, (t, h))]


def test_attention_pre_quant_validation_and_workspace(lib):
    from pypto_amd._runtime import AttentionPreQuantParams
    p = AttentionPreQuantParams(1e-5)
    # the quantised rows (256-byte aligned) + one int32 partial sum per 256 rows of the contraction
    assert lib.pto_attention_pre_quant_workspace(descs(apq_specs()), 19, ctypes.byref(p)) == 8 * 5120 + 20 * 8 * 1792 * 4
    assert lib.pto_attention_pre_quant_workspace(descs(apq_specs(t=3, h=256, q=128)), 19, ctypes.byref(p)) == 768 + 3 * 384 * 4
    rc, msg = launch_rc(lib, "attention_pre_quant", apq_specs(), p)
    assert rc == -5 and "workspace" in msg
    rc, msg = launch_rc(lib, "attention_pre_quant", apq_specs()[:18], p)
    assert rc == -1 and "19 tensors" in msg
    specs = apq_specs()
    specs[6] = (BF16, specs[6][1])
    rc, msg = launch_rc(lib, "attention_pre_quant", specs, p)
    assert rc == -2 and "atten_qkv_weight must be int8" in msg
    rc, msg = launch_rc(lib, "attention_pre_quant", apq_specs(h=5000), p)
    assert rc == -3 and "multiple of 256" in msg
    rc, msg = launch_rc(lib, "attention_pre_quant", apq_specs(d=64), p)
    assert rc == -3
    rc, msg = launch_rc(lib, "attention_pre_quant", apq_specs(half=65), p)
    assert rc == -3 and "half_rotary_dim" in msg
    specs = apq_specs()
    specs[16] = (BF16, (8, 256))          # key wider than value; widths no longer add up
    rc, msg = launch_rc(lib, "attention_pre_quant", specs, p)
    assert rc == -3
    specs = apq_specs()
    specs[13] = (BF16, (8, 32))
    rc, msg = launch_rc(lib, "attention_pre_quant", specs, p)
    assert rc == -3 and "cos must have rank 3" in msg
    assert launch_rc(lib, "attention_pre_quant", apq_specs(t=0), p)[0] == 0     # nothing to do, nothing launched
    assert launch_rc(lib, "attention_pre_quant", apq_specs(), AttentionPreQuantParams(float("nan")))[0] == -4


def test_paged_gather_validation(lib):
    from pypto_amd._runtime import PagedGatherParams
    INT64 = 4

    def specs(src=(INT8, (1024, 656)), idx=(INT32, (2, 16)), bt=(INT32, (2, 4)), out=(INT8, (32, 656))):
        return [src, idx, bt, out]
    p = PagedGatherParams(128, 0)
    assert lib.pto_paged_gather_workspace(descs(specs()), 4, ctypes.byref(p)) == 0
    rc, msg = launch_rc(lib, "paged_gather", specs()[:3], p)
    assert rc == -1 and "4 or 5 tensors" in msg
    rc, msg = launch_rc(lib, "paged_gather", specs(idx=(FP16, (2, 16))), p)
    assert rc == -2 and "indices must be int32 or int64" in msg
    rc, msg = launch_rc(lib, "paged_gather", specs(out=(FP16, (32, 656))), p)
    assert rc == -2 and "out must be int8" in msg
    rc, msg = launch_rc(lib, "paged_gather", specs(bt=(INT64, (3, 4))), p)
    assert rc == -3 and "block_table has 3 rows" in msg
    rc, msg = launch_rc(lib, "paged_gather", specs(out=(INT8, (31, 656))), p)
    assert rc == -3 and "out must be [32, 656]" in msg
    rc, msg = launch_rc(lib, "paged_gather", specs(out=(INT8, (32, 700))), PagedGatherParams(128, 700))
    assert rc == -4 and "exceeds the source row width" in msg
    assert launch_rc(lib, "paged_gather", specs(), PagedGatherParams(0, 0))[0] == -4
    assert launch_rc(lib, "paged_gather", specs(), PagedGatherParams(128, -1))[0] == -4
    rc, msg = launch_rc(lib, "paged_gather", specs() + [(INT32, (2,))], p)
    assert rc == -3 and "status must hold one word" in msg
    # nothing to gather: accepted, nothing launched
    assert launch_rc(lib, "paged_gather", specs(idx=(INT32, (2, 0)), out=(INT8, (0, 656))), p)[0] == 0
