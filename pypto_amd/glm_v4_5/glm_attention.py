"""Paged grouped-query decode attention of GLM-4.5.

Same entry points, argument order and semantics as the reference's models/glm_v4_5/glm_attention.py (``attention``
:1584-1622 and its per-SoC variants :1625-1700, ``check_args`` :45-63, ``IfaTileShapeConfig`` :66-73); the device code is
the gfx950 HIP kernel behind ``pto_gqa_decode_launch``.
"""
from dataclasses import dataclass, field

import torch

from .._runtime import GqaParams, launch
from ..error import FeError, PyptoError


@dataclass
class IfaTileShapeConfig:
    """Ascend tiling knobs of the reference operator; accepted for call compatibility and ignored."""
    g_tile: int = 12
    s2_tile: int = 1024
    c1_tile_shape: list = field(default_factory=list)
    v1_tile_shape: list = field(default_factory=list)
    c2_tile_shape: list = field(default_factory=list)
    v2_tile_shape: list = field(default_factory=list)


def check_args(query, key_cache, value_cache, block_tables, actual_seqs, attn_res):
    """The reference's argument assertions (glm_attention.py:45-63)."""
    assert query.dim() == 3
    assert query.dtype == torch.bfloat16
    assert key_cache.dim() == 4
    assert key_cache.dtype == torch.bfloat16
    assert value_cache.dim() == 4
    assert value_cache.dtype == torch.bfloat16
    assert block_tables.dim() == 2
    assert block_tables.dtype == torch.int32
    assert actual_seqs.dim() == 1
    assert actual_seqs.dtype == torch.int32
    assert attn_res.dim() == 3
    assert attn_res.dtype == torch.bfloat16


def attention(query, key_cache, value_cache, block_tables, actual_seqs, attn_res, softmax_scale, tile_config=None):
    """attn_res[t, h] = softmax(q[t, h] . K^T * softmax_scale) V over the first actual_seq - (s1 - 1 - j) cached tokens
    of the sequence (j = index of the query token within its sequence), K and V being KV head h // (nq // nkv) of the
    paged caches.  Written in place; returns None."""
    check_args(query, key_cache, value_cache, block_tables, actual_seqs, attn_res)
    try:
        launch("gqa_decode", [query, key_cache, value_cache, block_tables, actual_seqs, attn_res],
               GqaParams(float(softmax_scale), 0))
    except PyptoError:
        raise
    except Exception as e:  # noqa: BLE001 - everything is re-raised under the boundary's error type
        err = FeError(type(e)(f"Failed to call JIT function 'ifa_func_kernel'.\n{e}"))
        raise err.with_traceback(e.__traceback__) from None
    return None


# The reference keeps one entry per SoC / tuning flavour (glm_attention.py:1625-1700); they compute the same thing.
attention_for_950 = attention
attention_for_950_high_through = attention
attention_for_910_high_performance = attention
attention_for_910_s1_range_high_performance = attention
