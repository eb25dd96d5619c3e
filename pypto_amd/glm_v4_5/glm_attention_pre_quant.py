"""Fused attention prolog of GLM-4.5: residual add + RmsNorm, int8 quantisation, int8 QKV projection, head norms, rotary.

Same entry point, argument order and semantics as the reference's models/glm_v4_5/glm_attention_pre_quant.py
(``attention_pre_quant`` :633-747, ``check_args`` :50-129); the device code is the gfx950 HIP kernels behind
``pto_attention_pre_quant_launch``.  The weight is a plain row-major [hidden_size, total_head_size] int8 tensor (the
reference's "NZ" tiling is an Ascend device format).
"""
import torch

from .._runtime import AttentionPreQuantParams, launch
from ..error import FeError, PyptoError

EPS = 1e-05     # constant of the reference kernel (glm_attention_pre_quant.py:301)


def check_args(hidden_states, residual, input_layernorm_weight, input_layernorm_bias, atten_qkv_input_scale_reciprocal,
               atten_qkv_input_offset, atten_qkv_weight, atten_qkv_quant_bias, atten_qkv_deq_scale, atten_q_norm_weight,
               atten_q_norm_bias, atten_k_norm_weight, atten_k_norm_bias, cos, sin, query, key, value, residual_res):
    """The reference's argument assertions (glm_attention_pre_quant.py:50-129), less the Ascend storage formats."""
    bf = torch.bfloat16
    for t in (hidden_states, residual, query, key, value, residual_res):
        assert t.dim() == 2
        assert t.dtype == bf
    for t in (input_layernorm_weight, input_layernorm_bias, atten_qkv_input_scale_reciprocal, atten_qkv_input_offset,
              atten_q_norm_weight, atten_q_norm_bias, atten_k_norm_weight, atten_k_norm_bias):
        assert t.dim() == 1
        assert t.dtype == bf
    assert atten_qkv_weight.dim() == 2
    assert atten_qkv_weight.dtype == torch.int8
    assert atten_qkv_quant_bias.dim() == 1
    assert atten_qkv_quant_bias.dtype == torch.int32
    assert atten_qkv_deq_scale.dim() == 1
    assert atten_qkv_deq_scale.dtype == torch.float32
    for t in (cos, sin):
        assert t.dim() == 3
        assert t.shape[1] == 1
        assert t.dtype == bf


def attention_pre_quant(hidden_states, residual, input_layernorm_weight, input_layernorm_bias,
                        atten_qkv_input_scale_reciprocal, atten_qkv_input_offset, atten_qkv_weight, atten_qkv_quant_bias,
                        atten_qkv_deq_scale, atten_q_norm_weight, atten_q_norm_bias, atten_k_norm_weight,
                        atten_k_norm_bias, cos, sin, query, key, value, residual_res):
    """residual_res = hidden_states + residual; x = int8(rint(RmsNorm(residual_res) * scale + offset));
    [q | k | v] = bf16((x @ weight + quant_bias) * deq_scale); query = rotary(RmsNorm_q(q heads)),
    key = rotary(RmsNorm_k(k heads)) on each head's first 2 * cos.shape[-1] dims, value = v.  Every norm has a weight and
    a bias and epsilon 1e-5.  The four outputs are written in place; returns None."""
    tensors = [hidden_states, residual, input_layernorm_weight, input_layernorm_bias, atten_qkv_input_scale_reciprocal,
               atten_qkv_input_offset, atten_qkv_weight, atten_qkv_quant_bias, atten_qkv_deq_scale, atten_q_norm_weight,
               atten_q_norm_bias, atten_k_norm_weight, atten_k_norm_bias, cos, sin, query, key, value, residual_res]
    check_args(*tensors)
    try:
        launch("attention_pre_quant", tensors, AttentionPreQuantParams(EPS))
    except PyptoError:
        raise
    except Exception as e:  # noqa: BLE001 - everything is re-raised under the boundary's error type
        err = FeError(type(e)(f"Failed to call JIT function 'quant_attention_pre_kernel'.\n{e}"))
        raise err.with_traceback(e.__traceback__) from None
    return None
