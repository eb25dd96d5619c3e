"""Pins oracle.indexer_prolog: library routines, brute force and closed forms for every stage of the golden."""
import math

import torch

from oracle import indexer_prolog as op


def test_layer_norm_matches_the_library_routine():
    g = torch.Generator().manual_seed(1)
    x = torch.randn((5, 128), generator=g) * 3 + 1
    gamma = torch.randn(128, generator=g).to(torch.bfloat16)
    beta = torch.randn(128, generator=g).to(torch.bfloat16)
    ours = op.layer_norm(x, gamma, beta, 1e-6)
    ref = torch.nn.functional.layer_norm(x, (128,), gamma.float(), beta.float(), 1e-6)
    assert torch.allclose(ours, ref, rtol=1e-5, atol=1e-5)
    assert op.layer_norm(x.to(torch.bfloat16), gamma, beta).dtype == torch.bfloat16


def test_quant_int8_closed_form():
    g = torch.Generator().manual_seed(2)
    x = (torch.randn((7, 3, 128), generator=g) * 5).to(torch.bfloat16)
    y, s = op.quant_int8(x)
    assert y.dtype == torch.int8 and s.dtype == torch.float32 and s.shape == (7, 3, 1)
    mx = x.float().abs().amax(-1, keepdim=True)
    assert torch.equal(y.abs().amax(-1, keepdim=True).float(), torch.full_like(mx, 127))   # the largest maps to +-127
    assert torch.allclose(s, mx / 127, rtol=1e-6)
    assert ((y.float() * s - x.float()).abs() <= 0.5 * s * 1.0001).all()                     # nearest step
    # ties round to even: 0.5 steps -> 0, 1.5 steps -> 2
    t = torch.tensor([[127.0, 0.5, 1.5, 2.5, -0.5, -1.5]], dtype=torch.bfloat16)
    assert op.quant_int8(t)[0].tolist() == [[127, 0, 2, 2, 0, -2]]


def test_rope_rotates_pairs():
    g = torch.Generator().manual_seed(3)
    x = torch.randn((4, 2, 64), generator=g)
    ang = torch.rand((4, 64), generator=g) * 6.28
    ang[:, 32:] = ang[:, :32]                       # the same angle for both members of a pair (i, i + 32)
    y = op.single_rope(x, torch.cos(ang), torch.sin(ang))
    n_in = x[..., :32] ** 2 + x[..., 32:] ** 2
    n_out = y[..., :32] ** 2 + y[..., 32:] ** 2
    assert torch.allclose(n_in, n_out, rtol=1e-5, atol=1e-6)   # a rotation of each pair
    z = op.single_rope(x, torch.ones((4, 64)), torch.zeros((4, 64)))
    assert torch.equal(z, x)
    # quarter turn: (x1, x2) -> (-x2, x1)
    q = op.single_rope(x, torch.zeros((4, 64)), torch.ones((4, 64)))
    assert torch.equal(q[..., :32], -x[..., 32:]) and torch.equal(q[..., 32:], x[..., :32])


def test_int8_gemm_is_exact_and_scaled_in_order():
    c = op.make_case(2, 1, 256, seed=4, h=256, q_lora_rank=64, n=32)
    ref = (c["q_norm"].long() @ c["w_qb"].long())                          # brute force in int64
    assert ref.abs().max() < 2 ** 31
    q = (ref.float() * c["q_norm_scale"]) * c["w_qb_scale"].reshape(1, -1)
    c2 = dict(c, hadamard_q=torch.eye(128, dtype=torch.bfloat16), cos=torch.ones_like(c["cos"]), sin=torch.zeros_like(c["sin"]))
    qi, _ = op.intermediates(c2)                                           # identity rotary and hadamard: q passes through
    assert torch.equal(qi, q.reshape(2, 32, 128).to(torch.bfloat16))


def test_cache_scatter_touches_only_the_indexed_rows_and_weights_formula():
    c = op.make_case(3, 2, 300, seed=5, h=512, q_lora_rank=64, n=32)
    o = op.indexer_prolog(c)
    changed = (o["k_cache"].view(-1, 128) != c["k_cache"].view(-1, 128)).any(-1).nonzero().flatten()
    assert set(changed.tolist()) <= set(c["k_cache_index"].tolist()) and len(changed) >= 5
    rows = c["k_cache_index"]
    _, k = op.intermediates(c)
    ki, ks = op.quant_int8(k)
    assert torch.equal(o["k_cache"].view(-1, 128)[rows], ki)
    assert torch.equal(o["k_scale_cache"].view(-1)[rows], ks.to(torch.float16).view(-1))
    # the new tokens are the last s1 positions of each sequence
    bs = 128
    for i in range(3):
        for j in range(2):
            pos = 300 - 2 + j
            assert int(rows[i * 2 + j]) == int(c["block_table"][i, pos // bs]) * bs + pos % bs
    w = (c["x"].double() @ c["w_proj"].double())
    want = w.to(torch.bfloat16).float() * 32 ** -0.5 * 128 ** -0.5
    assert torch.allclose(o["weights"].float(), want, rtol=2 ** -9, atol=1e-6)


def test_walsh_hadamard_input_is_orthogonal():
    c = op.make_case(1, 1, 128, seed=6, h=256, q_lora_rank=64, n=32, hadamard="walsh")
    hm = c["hadamard_q"].float()
    assert torch.allclose(hm @ hm.t(), torch.eye(128), atol=1e-2)
    assert math.isclose(float(hm.abs().max()), 128 ** -0.5, rel_tol=1e-2)
