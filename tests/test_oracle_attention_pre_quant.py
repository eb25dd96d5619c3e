"""Pins the CPU oracle of GLM-4.5 attention_pre_quant (oracle/attention_pre_quant.py) without the reference at hand:
float64 closed forms, a complex-rotation identity, numpy integer arithmetic and hand-worked values, chosen so that a
dropped epsilon, a mean taken as a sum, a swapped rotary half, a wrong sign of sin, a transposed weight or a wrong split
order fails one of them.  The two NPU library calls of the reference golden (npu_quantize, npu_quant_matmul) cannot be
run here; for them the oracle follows the reference kernel's own arithmetic (glm_attention_pre_quant.py:389-407) and is
checked against that arithmetic done in numpy.
"""
import numpy as np
import torch

from oracle import attention_pre_quant as op

BF = torch.bfloat16


def bf16_close(a, b64, min_equal=0.98):
    """a (bf16) against a float64 value: within one bf16 step everywhere, equal to its rounding nearly everywhere."""
    a64 = a.double()
    assert ((a64 - b64).abs() <= 2.0 ** -7 * b64.abs() + 1e-30).all()
    assert (a == b64.to(BF)).double().mean() >= min_equal


def test_add_rms_norm_closed_form_and_epsilon():
    g = torch.Generator().manual_seed(1)
    for amp in (1.0, 1e-3):          # at 1e-3 the mean square (2e-6) is below the epsilon: dropping it shows
        x = (amp * torch.randn(5, 640, generator=g)).to(BF)
        r = (amp * torch.randn(5, 640, generator=g)).to(BF)
        gamma = (1 + 0.1 * torch.randn(640, generator=g)).to(BF)
        bias = (0.1 * torch.randn(640, generator=g)).to(BF)
        y, res = op.add_rms_norm(x, r, gamma, bias, 1e-5)
        s = x.double() + r.double()
        want = s / torch.sqrt((s * s).mean(-1, keepdim=True) + 1e-5) * gamma.double() + bias.double()
        bf16_close(y, want)
        assert torch.equal(res, s.float().to(BF))
        assert y.dtype == BF and res.dtype == BF
    # hand-worked: the row (3, 4) has mean square 12.5; gamma 2, bias 1
    y, res = op.add_rms_norm(torch.tensor([[1.0, 1.0]]).to(BF), torch.tensor([[2.0, 3.0]]).to(BF),
                             torch.tensor([2.0, 2.0]).to(BF), torch.tensor([1.0, 1.0]).to(BF), 0.0)
    assert torch.equal(res.float(), torch.tensor([[3.0, 4.0]]))
    want = torch.tensor([[6 / 12.5 ** 0.5 + 1, 8 / 12.5 ** 0.5 + 1]]).to(BF)
    assert torch.equal(y, want)


def test_rms_norm_bias_closed_form():
    g = torch.Generator().manual_seed(2)
    x = torch.randn(3, 4, 128, generator=g).to(BF)
    gamma = torch.rand(128, generator=g).to(BF)
    bias = torch.rand(128, generator=g).to(BF)
    y = op.rms_norm_bias(x, gamma, bias, 1e-5)
    xd = x.double()
    want = xd / torch.sqrt((xd * xd).mean(-1, keepdim=True) + 1e-5) * gamma.double() + bias.double()
    bf16_close(y, want)
    # every head is normalised on its own: scaling one head leaves it (almost) unchanged and the others untouched
    x2 = x.clone()
    x2[:, 1] = (x2[:, 1].float() * 4).to(BF)
    y2 = op.rms_norm_bias(x2, gamma, bias, 1e-5)
    assert torch.equal(y2[:, 0], y[:, 0]) and torch.equal(y2[:, 2:], y[:, 2:])
    assert (y2[:, 1].float() - y[:, 1].float()).abs().max() < 0.02


def test_quantize_rounding_offset_and_saturation():
    v = torch.tensor([[0.5, 1.5, 2.5, -0.5, -1.5, 300.0, -300.0, 1e6, -1e6, 126.5, 127.5, -128.5]]).to(BF)
    one, zero = torch.ones(12).to(BF), torch.zeros(12).to(BF)
    got = op.quantize(v, one, zero)
    assert got.dtype == torch.int8
    assert got.tolist() == [[0, 2, 2, 0, -2, 127, -128, 127, -128, 126, 127, -128]]
    # scale first, offset second: 3 * 2 + 1 = 7, not (3 + 1) * 2
    assert op.quantize(torch.tensor([[3.0]]).to(BF), torch.tensor([2.0]).to(BF), torch.tensor([1.0]).to(BF)).item() == 7
    # against numpy's rint on random rows (per-channel scale and offset)
    g = torch.Generator().manual_seed(3)
    x = torch.randn(4, 256, generator=g).to(BF)
    sc = (20 + 20 * torch.rand(256, generator=g)).to(BF)
    off = torch.round(5 * torch.randn(256, generator=g)).to(BF)
    want = np.clip(np.rint((x.float().numpy() * sc.float().numpy()).astype(np.float32) + off.float().numpy()), -128, 127)
    assert np.array_equal(op.quantize(x, sc, off).numpy(), want.astype(np.int8))


def test_quant_matmul_against_numpy_integers():
    g = torch.Generator().manual_seed(4)
    x = torch.randint(-128, 128, (6, 512), generator=g, dtype=torch.int8)
    w = torch.randint(-128, 128, (512, 96), generator=g, dtype=torch.int8)
    bias = torch.randint(-10 ** 6, 10 ** 6, (96,), generator=g, dtype=torch.int32)
    deq = torch.rand(96, generator=g).float()
    got = op.quant_matmul(x, w, bias, deq)
    acc = x.numpy().astype(np.int64) @ w.numpy().astype(np.int64) + bias.numpy().astype(np.int64)
    want = (acc.astype(np.float32) * deq.numpy()).astype(np.float32)            # int -> fp32 first, then the scale
    assert torch.equal(got, torch.from_numpy(want).to(BF))
    assert got.shape == (6, 96) and got.dtype == BF
    # a weight that picks channel j for output j (and nothing for a transposed reading): out = (x_j + bias_j) * deq_j
    w = torch.zeros(512, 96, dtype=torch.int8)
    w[torch.arange(96), torch.arange(96)] = 1
    got = op.quant_matmul(x, w, bias, deq)
    want = ((x[:, :96].int() + bias).float() * deq).to(BF)
    assert torch.equal(got, want)
    # sums beyond 2^24 are rounded to fp32 before the scale
    big = op.quant_matmul(torch.full((1, 4096), 127, dtype=torch.int8), torch.full((4096, 1), 127, dtype=torch.int8),
                          torch.tensor([1], dtype=torch.int32), torch.tensor([1.0]))
    assert big.item() == torch.tensor(float(np.float32(4096 * 127 * 127 + 1))).to(BF).item()


def test_rope_is_a_complex_rotation():
    g = torch.Generator().manual_seed(5)
    t, n, half = 5, 3, 32
    x = torch.randn(t, n, 2 * half, generator=g).to(BF)
    ang = torch.rand(t, 1, half, generator=g) * 6.28
    cos, sin = torch.cos(ang).to(BF), torch.sin(ang).to(BF)
    got = op.rope_half(x, cos, sin)
    z = torch.complex(x[..., :half].double(), x[..., half:].double()) * torch.complex(cos.double(), sin.double())
    want = torch.cat((z.real, z.imag), dim=-1)
    assert ((got.double() - want).abs() <= 2.0 ** -7 * want.abs() + 2.0 ** -9).all()
    assert (got == want.to(BF)).double().mean() > 0.95
    # quarter turn: (x1, x2) -> (-x2, x1); no turn: identity
    one, zero = torch.ones(t, 1, half).to(BF), torch.zeros(t, 1, half).to(BF)
    assert torch.equal(op.rope_half(x, zero, one), torch.cat((-x[..., half:], x[..., :half]), dim=-1))
    assert torch.equal(op.rope_half(x, one, zero), x)


def test_pipeline_order_and_split():
    inp = op.make_case(4, h=512, q_heads=3, kv_heads=2, d=128, half=32, seed=6)
    out = op.attention_pre_quant(inp)
    t, d, half = 4, 128, 32
    assert out["query"].shape == (t, 384) and out["key"].shape == (t, 256) and out["value"].shape == (t, 256)
    assert out["residual_res"].shape == (t, 512) and out["x_int8"].dtype == torch.int8
    x_norm, res = op.add_rms_norm(inp["hidden_states"], inp["residual"], inp["input_layernorm_weight"],
                                  inp["input_layernorm_bias"])
    assert torch.equal(out["residual_res"], res)
    xq = op.quantize(x_norm, inp["atten_qkv_input_scale_reciprocal"], inp["atten_qkv_input_offset"])
    assert torch.equal(out["x_int8"], xq)
    assert xq.float().abs().mean() > 10 and (xq.float().abs() == 127).float().mean() < 0.2   # the case uses the int8 range
    mm = op.quant_matmul(xq, inp["atten_qkv_weight"], inp["atten_qkv_quant_bias"], inp["atten_qkv_deq_scale"])
    # value = the last kv_size outputs, untouched; key = the kv_size before; query = the first q_size
    assert torch.equal(out["value"], mm[:, 384 + 256:])
    qn = op.rms_norm_bias(mm[:, :384].reshape(t, 3, d), inp["atten_q_norm_weight"], inp["atten_q_norm_bias"])
    kn = op.rms_norm_bias(mm[:, 384:640].reshape(t, 2, d), inp["atten_k_norm_weight"], inp["atten_k_norm_bias"])
    # the dims past the rotary part pass through
    assert torch.equal(out["query"].reshape(t, 3, d)[..., 2 * half:], qn[..., 2 * half:])
    assert torch.equal(out["key"].reshape(t, 2, d)[..., 2 * half:], kn[..., 2 * half:])
    assert torch.equal(out["query"].reshape(t, 3, d)[..., :2 * half], op.rope_half(qn[..., :2 * half], inp["cos"], inp["sin"]))
    assert torch.equal(out["key"].reshape(t, 2, d)[..., :2 * half], op.rope_half(kn[..., :2 * half], inp["cos"], inp["sin"]))
    # the key uses the key norm's weights, not the query's
    assert not torch.equal(kn, op.rms_norm_bias(mm[:, 384:640].reshape(t, 2, d), inp["atten_q_norm_weight"],
                                                inp["atten_q_norm_bias"]))
    tail = op.heads_from_x_int8(inp, xq)
    for k in ("query", "key", "value"):
        assert torch.equal(tail[k], out[k])


def test_reference_test_distribution_runs():
    """The reference test's own inputs (everything uniform in [0, 1): glm_attention_pre_quant.py:536-555) at its
    shape: 8 tokens, hidden 5120, 12 + 1 + 1 heads of 128."""
    inp = op.make_case(8, realistic=False, seed=7)
    out = op.attention_pre_quant(inp)
    assert out["query"].shape == (8, 1536) and out["key"].shape == (8, 128)
    for k in ("query", "key", "value", "residual_res"):
        assert torch.isfinite(out[k].float()).all()
