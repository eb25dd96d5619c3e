"""Pins oracle.mla_prolog: library routines, brute force and closed forms for every stage of the golden."""
import torch

from oracle import mla_prolog as op

SMALL = dict(h=512, q_lora_rank=256, n=4)


def test_rms_norm_matches_the_library_routine_and_the_epsilon_form():
    g = torch.Generator().manual_seed(1)
    x = torch.randn((5, 512), generator=g) * 3
    gamma = torch.randn(512, generator=g).to(torch.bfloat16)
    ref = torch.nn.functional.rms_norm(x, (512,), gamma.float(), 0.0)
    assert torch.allclose(op.rms_norm(x, gamma), ref, rtol=1e-5, atol=1e-6)
    ref = torch.nn.functional.rms_norm(x, (512,), gamma.float(), 1e-5)
    assert torch.allclose(op.rms_norm(x, gamma, 1e-5), ref, rtol=1e-5, atol=1e-6)
    # unit gamma: the result has unit root mean square
    y = op.rms_norm(x, torch.ones(512))
    assert torch.allclose((y * y).mean(-1), torch.ones(5), rtol=1e-5)
    assert op.rms_norm(x.to(torch.bfloat16), gamma).dtype == torch.bfloat16


def test_quant_closed_form_per_token_and_per_channel():
    g = torch.Generator().manual_seed(2)
    x = (torch.randn((7, 4, 128), generator=g) * 5).to(torch.bfloat16)
    y, s = op.quant(x)
    assert y.dtype == torch.int8 and s.dtype == torch.float32 and s.shape == (7, 4, 1)
    mx = x.float().abs().amax(-1, keepdim=True)
    assert torch.equal(y.abs().amax(-1, keepdim=True).float(), torch.full_like(mx, 127))
    assert torch.allclose(s, mx / 127, rtol=1e-6)
    assert ((y.float() * s - x.float()).abs() <= 0.5 * s * 1.0001).all()
    t = torch.tensor([[127.0, 0.5, 1.5, 2.5, -0.5, -1.5]], dtype=torch.bfloat16)
    assert op.quant(t)[0].tolist() == [[127, 0, 2, 2, 0, -2]]                 # ties to even
    w = torch.randn((64, 10), generator=g)
    yw, sw = op.quant(w, per_token=False)                                     # per output channel: over the rows
    assert sw.shape == (1, 10)
    assert torch.equal(yw.abs().amax(0).float(), torch.full((10,), 127.0))


def test_rope_is_a_complex_rotation_of_the_interleaved_pairs():
    g = torch.Generator().manual_seed(3)
    x = torch.randn((4, 3, 64), generator=g)
    ang = torch.rand((4, 32), generator=g) * 6.28
    cos = torch.cos(ang).repeat(1, 2)             # the same angle at positions i and 32 + i
    sin = torch.sin(ang).repeat(1, 2)
    y = op.rope_interleaved(x, cos, sin)
    z = torch.view_as_complex(x.reshape(4, 3, 32, 2).contiguous()) * torch.polar(torch.ones_like(ang), ang).unsqueeze(1)
    assert torch.allclose(y[..., :32], z.real, rtol=1e-5, atol=1e-6)
    assert torch.allclose(y[..., 32:], z.imag, rtol=1e-5, atol=1e-6)
    # no rotation: only the de-interleave remains
    y0 = op.rope_interleaved(x, torch.ones((4, 64)), torch.zeros((4, 64)))
    assert torch.equal(y0[..., :32], x[..., 0::2]) and torch.equal(y0[..., 32:], x[..., 1::2])
    # cos and sin are free per position (the golden does not tie position i to 32 + i)
    c, s = torch.randn((4, 64), generator=g), torch.randn((4, 64), generator=g)
    y = op.rope_interleaved(x, c, s)
    xe, xo = x[..., 0::2], x[..., 1::2]
    assert torch.allclose(y[..., :32], xe * c[:, None, :32] - xo * s[:, None, :32], rtol=1e-6, atol=1e-6)
    assert torch.allclose(y[..., 32:], xo * c[:, None, 32:] + xe * s[:, None, 32:], rtol=1e-6, atol=1e-6)


def test_query_path_against_brute_force():
    c = op.make_case(2, 1, 256, seed=4, **SMALL)
    out = op.mla_prolog(c)
    im = op.intermediates(c)
    # q_a: fp64 product rounded to bf16 (a bf16 step of slack for the fp32 accumulation)
    qa = c["x"].double() @ c["w_dq"].double()
    assert ((im["q_a"].double() - qa).abs() <= 2.0 ** -8 * qa.abs() + 1e-6).all()
    # quantised RmsNorm: dequantised values reproduce the normalised row to half a step
    deq = out["q_norm"].float() * out["q_norm_scale"]
    assert ((deq - im["q_rms"].float()).abs() <= 0.5 * out["q_norm_scale"] * 1.0001).all()
    # int8 GEMM exact (int64 brute force), scaled per token and per channel
    ref = out["q_norm"].long() @ c["w_uq_qr"].long()
    assert ref.abs().max() < 2 ** 31
    qb = ((ref.float() * out["q_norm_scale"]) * c["w_qb_scale"].reshape(1, -1)).to(torch.bfloat16).reshape(2, 4, 192)
    assert torch.equal(im["q_b"], qb)
    # q_nope: per-head product with w_uk, checked in fp64 by an einsum
    qn = torch.einsum("tnd,ndc->tnc", qb[..., :128].double(), c["w_uk"].double())
    assert ((out["q_nope"].double() - qn).abs() <= 2.0 ** -8 * qn.abs() + 1e-6).all()
    assert out["q_nope"].shape == (2, 4, 512) and out["q_rope"].shape == (2, 4, 64)
    assert torch.equal(out["q_rope"], op.rope_interleaved(qb[..., 128:], c["cos"], c["sin"]))


def test_key_path_and_cache_scatter():
    c = op.make_case(3, 2, 300, seed=5, **SMALL)
    out = op.mla_prolog(c)
    im = op.intermediates(c)
    rows = c["cache_index"]
    t = rows.numel()
    assert len(set(rows.tolist())) == t
    # the last s1 positions of each sequence, through the page table
    table = c["block_table"]
    for i in range(3):
        for j in range(2):
            pos = 300 - 2 + j
            assert int(rows[i * 2 + j]) == int(table[i, pos // 128]) * 128 + pos % 128
    kv, ks, kr = out["kv_cache"].view(-1, 512), out["k_scale_cache"].view(-1, 4), out["kr_cache"].view(-1, 64)
    # dequantised cache rows reproduce the normalised key to half a step of their group
    deq = (kv[rows].float().reshape(t, 4, 128) * ks[rows].reshape(t, 4, 1)).reshape(t, 512)
    step = ks[rows].repeat_interleave(128, dim=1)
    assert ((deq - im["kv_rms"].float()).abs() <= 0.5 * step * 1.0001).all()
    assert torch.equal(kv[rows].reshape(t, 4, 128).abs().amax(-1).float(), torch.full((t, 4), 127.0))
    assert torch.equal(kr[rows], op.rope_interleaved(im["kv"][:, 512:].reshape(t, 1, 64), c["cos"], c["sin"]).reshape(t, 64))
    # nothing but the indexed rows changes
    keep = torch.ones(kv.shape[0], dtype=torch.bool)
    keep[rows] = False
    assert torch.equal(kv[keep], c["kv_cache"].view(-1, 512)[keep])
    assert torch.equal(ks[keep], c["k_scale_cache"].view(-1, 4)[keep])
    assert torch.equal(kr[keep], c["kr_cache"].view(-1, 64)[keep])


def test_epsilon_form_is_within_the_reference_tolerance_of_the_golden():
    c = op.make_case(2, 2, 256, seed=6, **SMALL)
    a, b = op.mla_prolog(c), op.mla_prolog(c, 1e-5, 1e-5)
    assert (a["q_norm"].int() - b["q_norm"].int()).abs().max() <= 1
    assert torch.allclose(a["q_norm_scale"], b["q_norm_scale"], rtol=5e-3, atol=2.5e-5)
    assert (a["kv_cache"].int() - b["kv_cache"].int()).abs().max() <= 1


def test_bf16_form_has_no_quantisation_anywhere():
    c = op.make_case(3, 2, 300, seed=7, quant_b=False, **SMALL)
    assert c["w_uq_qr"].dtype == torch.bfloat16 and c["w_qb_scale"].numel() == 0 and c["kv_cache"].dtype == torch.bfloat16
    out = op.mla_prolog(c)
    im = op.intermediates(c)
    rows = c["cache_index"]
    t = rows.numel()
    assert out["q_norm_scale"] is None and torch.equal(out["q_norm"], im["q_rms"])           # q_norm is the RmsNorm output
    qb = (im["q_rms"].double() @ c["w_uq_qr"].double()).reshape(t, 4, 192)                    # fp64 product, bf16 slack
    assert ((im["q_b"].double() - qb).abs() <= 2.0 ** -8 * qb.abs() + 1e-6).all()
    qn = torch.einsum("tnd,ndc->tnc", im["q_b"][..., :128].double(), c["w_uk"].double())
    assert ((out["q_nope"].double() - qn).abs() <= 2.0 ** -8 * qn.abs() + 1e-6).all()
    assert torch.equal(out["q_rope"], op.rope_interleaved(im["q_b"][..., 128:], c["cos"], c["sin"]))
    kv = out["kv_cache"].view(-1, 512)
    assert torch.equal(kv[rows], im["kv_rms"])                                                # the cache row is the normalised key
    assert torch.equal(out["k_scale_cache"], c["k_scale_cache"])                              # scales untouched
    keep = torch.ones(kv.shape[0], dtype=torch.bool)
    keep[rows] = False
    assert torch.equal(kv[keep], c["kv_cache"].view(-1, 512)[keep])
