"""Sparse flash attention over the int8 paged MLA cache, packed 656-byte cache rows.

Same entry points, argument order and semantics as the reference module
models/deepseek_v32_exp/sparse_attention_antiquant_impl.py (``SaTileShapeConfig`` :34-41,
``sparse_attention_antiquant_d`` :287-302, ``_p`` :358-373, ``_d_950`` :739-749).  A cache row is
512 int8 nope | 64 bf16 rope | 4 fp32 scales; ``attention_out`` is 2-D ``[t * nq, 512]``.
"""
from dataclasses import dataclass, field

from .._runtime import SfaParams, launch, operator


@dataclass
class SaTileShapeConfig:
    """Ascend tiling knobs of the reference operator; accepted for call compatibility and ignored."""
    g_tile: int = 128
    s_kv_tile: int = 2048
    c1_tile_shape: list = field(default_factory=list)
    v1_tile_shape: list = field(default_factory=list)
    c2_tile_shape: list = field(default_factory=list)
    v2_tile_shape: list = field(default_factory=list)


_SCALARS = ("nq", "n_kv", "softmax_scale", "topk", "block_size", "max_blocknum_perbatch", "tile_config")


def _run(query_nope, query_rope, nope_cache, topk_indices, block_table, kv_act_seqs, attention_out, nq, n_kv,
         softmax_scale, topk, block_size, max_blocknum_perbatch, tile_config):
    params = SfaParams(int(nq), int(n_kv), float(softmax_scale), int(topk), int(block_size),
                       int(max_blocknum_perbatch), 0)
    launch("sfa_antiquant", [query_nope, query_rope, nope_cache, topk_indices, block_table, kv_act_seqs,
                             attention_out], params)


@operator(7, _SCALARS)
def sparse_attention_antiquant_d(*tensors, **scalars):
    _run(*tensors, **scalars)


@operator(7, _SCALARS)
def sparse_attention_antiquant_p(*tensors, **scalars):
    _run(*tensors, **scalars)


@operator(7, _SCALARS)
def sparse_attention_antiquant_d_950(*tensors, **scalars):
    _run(*tensors, **scalars)
