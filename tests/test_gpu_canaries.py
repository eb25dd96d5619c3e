"""Out-of-bounds-write detection without a GPU sanitizer: every operand and the workspace of a call are carved out of
larger buffers filled with a sentinel, the operator runs on the carved copies through the C ABI, and every sentinel byte
in front of and behind each region must be intact afterwards (the place of the reference's GM out-of-bounds check,
python/pypto/config.py:536-537).  The shapes end inside the kernels' tiles (token counts, head counts, list lengths,
row widths that are not multiples of a tile), which is where a store past the end would come from.  Host-side checks
only: nothing here can provoke a fault - a store that strays lands in the guard area of an allocation.

The operators are called through their ordinary Python entry points; a fixture swaps the launch function for one that
makes the carved copies, launches through the ctypes binding with a carved workspace of exactly the size the workspace
query returns, checks the guards and copies the results back.  Results must equal an ordinary call's bit for bit."""
import ctypes
import importlib

import pytest
import torch

from pypto_amd import _runtime

pytestmark = pytest.mark.gpu

GUARD = 4096  # bytes of sentinel on either side of a region (a multiple of 256: the regions stay aligned like allocations)
SENTINEL = 0xA5
MODULES = ["pypto_amd.deepseek_v32_exp.lightning_indexer_prolog_quant_impl", "pypto_amd.deepseek_v32_exp.lightning_indexer_quant_impl",
           "pypto_amd.deepseek_v32_exp.mla_indexer_prolog_quant_impl", "pypto_amd.deepseek_v32_exp.mla_prolog_quant_impl",
           "pypto_amd.deepseek_v32_exp.sparse_attention_antiquant_impl", "pypto_amd.deepseek_v32_exp.sparse_flash_attention_quant_impl",
           "pypto_amd.experimental.gather", "pypto_amd.glm_v4_5.glm_attention", "pypto_amd.glm_v4_5.glm_attention_pre_quant",
           "pypto_amd.glm_v4_5.glm_select_experts"]


class Carved:
    def __init__(self, nbytes, dev):
        self.nbytes = nbytes
        self.buf = torch.full((GUARD + nbytes + GUARD,), SENTINEL, dtype=torch.uint8, device=dev)
        self.region = self.buf[GUARD:GUARD + nbytes]

    def intact(self):
        return bool((self.buf[:GUARD] == SENTINEL).all()) and bool((self.buf[GUARD + self.nbytes:] == SENTINEL).all())


def install_guards(monkeypatch):
    """Routes every operator launch through carved operands and a carved workspace; returns the log of launches."""
    log = []

    def launch(op, tensors, params):
        carved, views = {}, []
        for t in tensors:
            key = (t.data_ptr(), t.dtype, tuple(t.shape))  # (a cache passed as input and as output is one region)
            if key not in carved:
                c = Carved(t.numel() * t.element_size(), t.device)
                view = c.region.view(t.dtype).view(t.shape) if t.numel() else t
                if t.numel():
                    view.copy_(t)
                carved[key] = (c, view, t)
            views.append(carved[key][1])
        lib = _runtime.load_library()
        n = getattr(lib, f"pto_{op}_workspace")(_runtime.describe(views), len(views), ctypes.byref(params))
        ws = Carved(int(n), views[0].device)
        _runtime.launch_ctypes(op, views, params, workspace=ws.region if n else None, sync=1)
        torch.cuda.synchronize()
        assert ws.intact(), f"{op}: a store outside the workspace ({n} bytes)"
        for i, (c, view, t) in enumerate(carved.values()):
            assert c.intact(), f"{op}: a store outside operand {i} {tuple(t.shape)} {t.dtype}"
            if t.numel():
                t.copy_(view)
        log.append((op, int(n)))

    # (the operator modules first: one imported while _runtime.launch is swapped would bind the swapped function for good)
    modules = [importlib.import_module(name) for name in MODULES]
    monkeypatch.setattr(_runtime, "launch", launch)
    for m in modules:
        monkeypatch.setattr(m, "launch", launch)
    return log


@pytest.fixture
def guarded(monkeypatch, cuda):
    return install_guards(monkeypatch)


def test_sparse_flash_attention(cuda, guarded):
    from oracle import sfa as osfa
    from _cases import run_sfa
    # 48 heads (a partly filled head group), lists that end inside a 32-row tile, an empty and a one-entry list,
    # several KV splits (workspace in use) and the packed-row entry
    for kw, packed, entry in ((dict(b=3, nq=48, s1=2, act=[700, 33, 2053], topk=1024), False, "d"),
                              (dict(b=2, nq=128, s1=1, act=[5000, 1], topk=2048), True, "d_950"),
                              (dict(b=1, nq=200, s1=3, act=[77], topk=64), False, "p")):
        case = osfa.make_case(kw["b"], kw["nq"], kw["s1"], kw["act"], topk=kw["topk"], seed=31, dist="bench", softmax_scale=192 ** -0.5)
        got = run_sfa(case, cuda, entry=entry, packed=packed)
        assert guarded and guarded[-1][0] in ("sfa_quant", "sfa_antiquant")
    assert any(n > 0 for _, n in guarded), "at least one case must use KV splits"
    assert torch.isfinite(got.float()).all()


def test_sparse_flash_attention_equals_the_ordinary_call(cuda):
    from oracle import sfa as osfa
    from _cases import run_sfa
    case = osfa.make_case(3, 48, 2, [700, 33, 2053], topk=1024, seed=31, dist="bench", softmax_scale=192 ** -0.5)
    plain = run_sfa(case, cuda)
    mp = pytest.MonkeyPatch()
    try:
        log = install_guards(mp)
        assert torch.equal(run_sfa(case, cuda), plain) and log
    finally:
        mp.undo()


def test_lightning_indexer(cuda, guarded):
    from oracle import indexer as oi
    from _cases import run_indexer
    from test_gpu_indexer import check_topk
    # lengths that end inside a 2048-key span, a 128-key page and a 64-key group; fewer keys than the selection; none
    for b, s1, act, seed in ((4, 2, [5000, 700, 129, 0], 41), (3, 1, [2049, 4095, 64], 42), (2, 3, [9000, 3], 43)):
        case = oi.make_case(b, s1, act, seed=seed)
        check_topk(case, run_indexer(case, cuda))
    assert all(op == "lightning_indexer" and n > 0 for op, n in guarded)


def test_topk(cuda, guarded):
    from pypto_amd.op import topk
    from oracle import topk as otopk
    g = torch.Generator().manual_seed(6)
    for shape, k in (((7, 300), 50), ((3, 8193), 2048), ((2, 20000), 1000), ((5, 3), 3), ((1, 1), 1)):
        x = torch.randn(shape, generator=g)
        vals, idx = topk(x.to(cuda), k)
        gv, gi = otopk.topk_rows(x, k, True)
        assert torch.equal(idx.cpu(), gi) and torch.equal(vals.cpu(), gv)
    assert len(guarded) == 5


def test_paged_gather(cuda, guarded):
    from pypto_amd.experimental import gather_in_l1, gather_in_ub
    from oracle import paged
    g = torch.Generator().manual_seed(7)
    # row widths that take the 16-, 4-, 2- and 1-byte copy paths, index counts that end inside a 32-row workgroup
    for hidden, size, bs, nblk, k, dtype in ((656, 656, 16, 40, 77, torch.int8), (36, 20, 4, 13, 33, torch.float32),
                                             (7, 7, 3, 5, 15, torch.bfloat16), (129, 1, 8, 6, 41, torch.int8)):
        n = nblk * bs
        src = torch.randint(-100, 100, (n, hidden), generator=g).to(dtype)
        page = torch.randperm(nblk, generator=g).to(torch.int32).reshape(1, nblk)
        idx = torch.randint(0, n, (1, k), generator=g, dtype=torch.int32)
        if size != hidden:   # the first `size` columns of every row
            out = gather_in_l1(src.to(cuda), idx.to(cuda), page.to(cuda), bs, size).cpu()
        else:
            out = gather_in_ub(src.to(cuda), idx.to(cuda), page.to(cuda), bs, -2).cpu()
        want = paged.paged_gather(src, idx[0], page[0], bs)[:, :size]
        assert torch.equal(out.view(torch.uint8), want.contiguous().view(torch.uint8))
    assert len(guarded) == 4


def test_indexer_prolog(cuda, guarded):
    from oracle import indexer_prolog as op
    from test_gpu_indexer_prolog import check, run
    # token counts inside a 32-token tile (decode kernels) and inside a 128-token tile (prefill kernels)
    for b, s1, seed, kw in ((5, 1, 51, dict(h=1024, q_lora_rank=256, n=32)), (3, 3, 52, {}), (43, 3, 53, dict(h=1024, q_lora_rank=256, n=32))):
        case = op.make_case(b, s1, 600, seed=seed, **kw)
        check(case, run(case, cuda))
    assert all(o == "indexer_prolog" for o, _ in guarded) and len(guarded) == 3


def test_mla_prolog(cuda, guarded):
    from oracle import mla_prolog as op
    from test_gpu_mla_prolog import check, check_bf16_form, run
    for b, s1, seed, kw in ((37, 1, 61, dict(h=512, q_lora_rank=256, n=4)), (3, 2, 62, dict(h=1024, q_lora_rank=384, n=6)),
                            (130, 1, 63, dict(h=512, q_lora_rank=256, n=4))):
        case = op.make_case(b, s1, 300, seed=seed, **kw)
        check(case, run(case, cuda, entry="mla_prolog_quant_p" if b >= 128 else "mla_prolog_quant_d"))
    case = op.make_case(5, 1, 300, seed=64, h=512, q_lora_rank=256, n=4, quant_b=False)
    check_bf16_form(case, run(case, cuda))
    assert all(o == "mla_prolog_quant" for o, _ in guarded) and len(guarded) == 4


def test_mla_indexer_prolog(cuda, guarded):
    from oracle import mla_prolog as op
    from test_gpu_mla_indexer_prolog import check_against_oracle, run_fused
    for b, s1, seed in ((5, 1, 71), (3, 2, 72), (131, 1, 73)):
        mla_case, idx_case = op.make_fused_case(b, s1, 600, seed=seed, n_idx=64, h=512, q_lora_rank=256, n=4)
        got = run_fused(mla_case, idx_case, cuda, entry="mla_indexer_prolog_quant_p" if b >= 128 else "mla_indexer_prolog_quant_d")
        check_against_oracle(mla_case, idx_case, got)
    assert all(o == "mla_indexer_prolog_quant" for o, _ in guarded) and len(guarded) == 3


def test_secondary_operators(cuda, guarded):
    """GLM-4.5 expert selection, paged GQA decode and attention_pre_quant under the same guards."""
    from oracle import gqa as og
    from test_gpu_gqa import check as check_gqa, run as run_gqa
    from test_gpu_select_experts import check as check_se
    from oracle import select_experts as ose
    case = og.make_case(3, 2, 12, 1, [300, 2049, 77], seed=81)
    check_gqa(run_gqa(case, cuda), case, "guarded gqa")
    logits, bias = ose.make_case(1027, 160, seed=82)
    check_se(logits, bias, 8, True, 4, 8, cuda, scale=2.5)
    assert {o for o, _ in guarded} >= {"gqa_decode", "select_experts"}
