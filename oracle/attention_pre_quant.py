"""CPU restatement of the reference's GLM-4.5 ``attention_pre_quant`` (test infrastructure only).

The producer of the query / key / value rows the GLM-4.5 paged attention reads: residual add + RmsNorm with bias,
per-channel int8 quantisation of the normalised row, int8 QKV projection with an int32 bias and per-output fp32
dequantisation, per-head RmsNorm with bias on the query and key heads, rotary embedding on the first ``2 * half`` dims
of every query and key head.

Follows the reference operator's own arithmetic, step by step, in models/glm_v4_5/glm_attention_pre_quant.py
(``quant_attention_pre_kernel`` :235-505, helpers ``rms_norm_bias`` :188-218 and ``rope_data`` :221-231) and the
torch golden beside it (``add_rms_norm_npu_golden`` :133-147, ``rms_norm_npu_golden`` :150-162,
``apply_rotary_pos_emb_v2`` :173-185; assembled at :591-619 and in utils/golden/attn_golden.py:324-378).

Parity unpinned for two steps: the golden quantises and multiplies with two NPU library calls
(``torch_npu.npu_quantize``, ``torch_npu.npu_quant_matmul``, :594-595) that do not exist here and whose outputs the
reference holds no fixture of.  For those two steps this file follows what the reference *kernel* computes
(:389-407): ``int8(sat(rint(bf16_norm * scale + offset)))`` and ``bf16(float(int32 sum + int32 bias) * deq_scale)``;
whether the NPU library rounds the same way cannot be checked in this build.  Everything else is pinned by
tests/test_oracle_attention_pre_quant.py against float64 closed forms, a complex-rotation identity, numpy integer
arithmetic and hand-worked special cases.
"""
import torch

EPS = 1e-5      # the kernel's constant (:301)


def add_rms_norm(x, residual, gamma, bias, eps=EPS):
    """:361-386 / golden :133-147 - returns (bf16 normalised row, bf16 sum row).  fp32 throughout: sum, square, times
    1/h, row sum + eps, sqrt, divide, times gamma, plus bias; the two results are rounded to bf16 separately."""
    xf = residual.float() + x.float()
    h = x.shape[-1]
    mean = (xf * xf) * (1.0 / h)
    denom = torch.sqrt(torch.sum(mean, dim=-1, keepdim=True) + eps)
    y = (xf / denom) * gamma.float() + bias.float()
    return y.to(torch.bfloat16), xf.to(torch.bfloat16)


def rms_norm_bias(x, gamma, bias, eps=EPS):
    """:188-218 / golden :150-162 - over the last dim, result in x's dtype."""
    xf = x.float()
    mean = (xf * xf) * (1.0 / x.shape[-1])
    denom = torch.sqrt(torch.sum(mean, dim=-1, keepdim=True) + eps)
    return ((xf / denom) * gamma.float() + bias.float()).to(x.dtype)


def quantize(x_norm, scale, offset):
    """:389-396 - bf16 row -> fp32, times the per-channel scale, plus the per-channel offset (two roundings), round to
    nearest even to int32, through fp16 to int8 with saturation: every int32 beyond the int8 range, however large,
    ends at -128 or 127 (fp16 turns what it cannot hold into an infinity of the right sign)."""
    v = x_norm.float() * scale.float() + offset.float()
    return torch.clamp(torch.round(v), -128, 127).to(torch.int8)


def quant_matmul(x_int8, weight, quant_bias, deq_scale):
    """:398-403 - exact int32 product, + int32 bias, -> fp32 (round to nearest even beyond 2^24), times the per-output
    scale, -> bf16."""
    # the integer product through float64 BLAS: every partial sum is an integer below 2^53, so it is exact
    acc = torch.matmul(x_int8.double(), weight.double()).to(torch.int64) + quant_bias.to(torch.int64)
    return (acc.to(torch.int32).float() * deq_scale.float()).to(torch.bfloat16)


def rope_half(x_rot, cos, sin):
    """:446-473, ``rope_data`` :221-231 / golden :165-185 - x_rot [t, heads, 2 * half] bf16, cos / sin [t, 1, half];
    (x1, x2) = the two halves; o1 = x1 cos - x2 sin, o2 = x2 cos + x1 sin in fp32 (each product and sum rounded),
    -> bf16."""
    xf = x_rot.float()
    c, s = cos.float(), sin.float()
    x1, x2 = torch.chunk(xf, 2, dim=-1)
    o1 = x1 * c - x2 * s
    o2 = x2 * c + x1 * s
    return torch.cat((o1, o2), dim=-1).to(x_rot.dtype)


def attention_pre_quant(inp, eps=EPS):
    """inp: the operator's input tensors by the names of the reference signature (:634-654) plus ``q_size`` and
    ``kv_size``.  Returns query [t, q_size], key [t, kv_size], value [t, kv_size], residual_res [t, h] (bf16) and the
    intermediate int8 row ``x_int8`` [t, h]."""
    x_norm, residual_res = add_rms_norm(inp["hidden_states"], inp["residual"], inp["input_layernorm_weight"],
                                        inp["input_layernorm_bias"], eps)
    x_int8 = quantize(x_norm, inp["atten_qkv_input_scale_reciprocal"], inp["atten_qkv_input_offset"])
    out = heads_from_x_int8(inp, x_int8, eps)
    out.update(residual_res=residual_res, x_int8=x_int8)
    return out


def heads_from_x_int8(inp, x_int8, eps=EPS):
    """Everything after the quantisation, from a given int8 row: what the stages downstream of the first kernel must
    produce exactly."""
    d = inp["atten_q_norm_weight"].shape[0]
    half = inp["cos"].shape[-1]
    q_size, kv_size = inp["q_size"], inp["kv_size"]
    t = x_int8.shape[0]
    mm = quant_matmul(x_int8, inp["atten_qkv_weight"], inp["atten_qkv_quant_bias"], inp["atten_qkv_deq_scale"])
    q, k, v = mm.split([q_size, kv_size, kv_size], dim=-1)                                        # :410-425
    q = rms_norm_bias(q.reshape(t, q_size // d, d), inp["atten_q_norm_weight"], inp["atten_q_norm_bias"], eps)
    k = rms_norm_bias(k.reshape(t, kv_size // d, d), inp["atten_k_norm_weight"], inp["atten_k_norm_bias"], eps)
    q = torch.cat((rope_half(q[..., :2 * half], inp["cos"], inp["sin"]), q[..., 2 * half:]), dim=-1)
    k = torch.cat((rope_half(k[..., :2 * half], inp["cos"], inp["sin"]), k[..., 2 * half:]), dim=-1)
    return {"query": q.reshape(t, q_size), "key": k.reshape(t, kv_size), "value": v.contiguous()}


def make_case(t, h=5120, q_heads=12, kv_heads=1, d=128, half=32, seed=0, realistic=True):
    """Synthetic inputs.  ``realistic=False``: the reference test's own distributions (:536-555: everything
    torch.rand, int8 weights uniform over the whole range, bias in [-128, 128), which saturates most of the int8 row);
    ``realistic=True``: zero-mean activations, gamma near 1, a quantisation scale that spreads the normalised row over
    the int8 range, cos / sin of real angles."""
    g = torch.Generator().manual_seed(seed)
    bf = torch.bfloat16
    n_out = (q_heads + 2 * kv_heads) * d

    def rand(*s):
        return torch.rand(*s, generator=g)

    def randn(*s):
        return torch.randn(*s, generator=g)

    if realistic:
        ang = rand(t, 1, half) * 6.2831853
        inp = {
            "hidden_states": randn(t, h).to(bf), "residual": randn(t, h).to(bf),
            "input_layernorm_weight": (1 + 0.1 * randn(h)).to(bf), "input_layernorm_bias": (0.05 * randn(h)).to(bf),
            "atten_qkv_input_scale_reciprocal": (30 + 10 * rand(h)).to(bf),
            "atten_qkv_input_offset": torch.round(4 * randn(h)).to(bf),
            "atten_qkv_deq_scale": (1e-4 * (0.5 + rand(n_out))).float(),
            "atten_q_norm_weight": (1 + 0.1 * randn(d)).to(bf), "atten_q_norm_bias": (0.05 * randn(d)).to(bf),
            "atten_k_norm_weight": (1 + 0.1 * randn(d)).to(bf), "atten_k_norm_bias": (0.05 * randn(d)).to(bf),
            "cos": torch.cos(ang).to(bf), "sin": torch.sin(ang).to(bf),
        }
    else:
        inp = {
            "hidden_states": rand(t, h).to(bf), "residual": rand(t, h).to(bf),
            "input_layernorm_weight": rand(h).to(bf), "input_layernorm_bias": rand(h).to(bf),
            "atten_qkv_input_scale_reciprocal": rand(h).to(bf), "atten_qkv_input_offset": rand(h).to(bf),
            "atten_qkv_deq_scale": rand(n_out).float(),
            "atten_q_norm_weight": rand(d).to(bf), "atten_q_norm_bias": rand(d).to(bf),
            "atten_k_norm_weight": rand(d).to(bf), "atten_k_norm_bias": rand(d).to(bf),
            "cos": rand(t, 1, half).to(bf), "sin": rand(t, 1, half).to(bf),
        }
    inp["atten_qkv_weight"] = torch.randint(-128, 128, (h, n_out), generator=g, dtype=torch.int8)
    inp["atten_qkv_quant_bias"] = torch.randint(-128, 128, (n_out,), generator=g, dtype=torch.int32)
    inp["q_size"] = q_heads * d
    inp["kv_size"] = kv_heads * d
    return inp
