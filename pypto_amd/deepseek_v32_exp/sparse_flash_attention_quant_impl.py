"""Sparse flash attention over the int8 paged MLA cache, three-tensor cache layout.

Same entry points, argument order and semantics as the reference module
models/deepseek_v32_exp/sparse_flash_attention_quant_impl.py (``SaTileShapeConfig`` :34-42,
``sparse_flash_attention_quant_d_950`` :572-591, ``_d`` :655-674, ``_p`` :734-753); the device code is
the gfx950 HIP kernel behind ``pto_sfa_quant_launch``.
"""
from dataclasses import dataclass, field

from .._runtime import SfaParams, launch, operator


@dataclass
class SaTileShapeConfig:
    """Ascend tiling knobs of the reference operator; accepted for call compatibility and ignored."""
    g_tile: int = 128
    s_kv_tile: int = 2048
    gather_vec_tile_shape: list = field(default_factory=list)
    c1_tile_shape: list = field(default_factory=list)
    v1_tile_shape: list = field(default_factory=list)
    c2_tile_shape: list = field(default_factory=list)
    v2_tile_shape: list = field(default_factory=list)


_SCALARS = ("nq", "n_kv", "softmax_scale", "topk", "block_size", "max_blocknum_perbatch", "tile_config")


def _run(query_nope, query_rope, key_nope_2d, key_rope_2d, k_nope_scales, topk_indices, block_table, kv_act_seqs,
         attention_out, nq, n_kv, softmax_scale, topk, block_size, max_blocknum_perbatch, tile_config):
    params = SfaParams(int(nq), int(n_kv), float(softmax_scale), int(topk), int(block_size),
                       int(max_blocknum_perbatch), 0)
    launch("sfa_quant", [query_nope, query_rope, key_nope_2d, key_rope_2d, k_nope_scales, topk_indices, block_table,
                         kv_act_seqs, attention_out], params)


@operator(9, _SCALARS)
def sparse_flash_attention_quant_d(*tensors, **scalars):
    """Decode entry: attention_out[b, s1, nq, 512] = softmax(q K_sel^T * scale) V_sel per query token."""
    _run(*tensors, **scalars)


@operator(9, _SCALARS)
def sparse_flash_attention_quant_d_950(*tensors, **scalars):
    """Decode entry (the reference's second SoC flavour); same computation."""
    _run(*tensors, **scalars)


@operator(9, _SCALARS)
def sparse_flash_attention_quant_p(*tensors, **scalars):
    """Prefill entry (s1 > 1 query tokens per sequence); same computation."""
    _run(*tensors, **scalars)
