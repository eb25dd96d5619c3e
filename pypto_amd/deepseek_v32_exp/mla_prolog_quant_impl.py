"""MLA prolog: hidden states -> the attention query (q_nope, q_rope), the quantised normalised query that
the lightning-indexer prolog reads (q_norm, q_norm_scale) and the new rows of the paged int8 MLA cache
(kv_cache, k_scale_cache, kr_cache) that sparse flash attention reads.

Same entry points, dataclasses, argument order and semantics as the reference module
models/deepseek_v32_exp/mla_prolog_quant_impl.py (``MlaTileConfig`` :57-75, ``MlaQuantInputs`` :78-86,
``RopeTileShapeConfig`` :89-93, ``mla_prolog_quant_p`` :745-842, ``mla_prolog_quant_d`` :845-951); the device code is
the gfx950 HIP kernels behind ``pto_mla_prolog_quant_launch``.  The weights are taken in plain row-major layout (the
reference casts w_dq, w_uq_qr and w_dkv_kr to the Ascend NZ tiling, a device format, before the call).  Both forms of
the reference: int8 (w_uq_qr INT8 with its dequant_scale, q_norm_out and kv_cache INT8 with FP32 scales) and bf16 (an
empty dequant_scale; w_uq_qr, q_norm_out and kv_cache BF16, the scale tensors left alone).
"""
from dataclasses import dataclass, field
from typing import List

import torch

from .._runtime import MlaPrologParams, launch, operator


class MlaTileConfig:
    """Ascend tiling knobs of the reference operator; accepted for call compatibility and ignored."""

    def __init__(self):
        self.tile_b = 8
        self.tile_s = 1
        self.tile_bs = 8
        self.m_tile = 16
        self.mv_tile = 16
        self.pre_quant_cube_tile = [16, 16, 256, 256, 128, 128]
        self.cube_qb_tile = [16, 16, 256, 256, 128, 128]
        self.cube_wuk_tile = [32, 32, 256, 256, 256, 256]
        self.unroll_list = [32, 16, 8, 4, 2, 1]
        self.q_vec_tile0 = 16
        self.q_vec_tile1 = 16
        self.k_vec_tile0 = 16
        self.k_vec_tile1 = 16
        self.cube_l1_reuse_setting = {-1: 4}
        self.cube_nbuffer_setting = {3: 4}
        self.dynamic_unaligned_enable = False


@dataclass
class MlaQuantInputs:
    dequant_scale_x: torch.Tensor = None
    dequant_scale_w_dq: torch.Tensor = None
    dequant_scale_w_uq_qr: torch.Tensor = None
    dequant_scale_w_dkv_kr: torch.Tensor = None
    quant_scale_ckv: torch.Tensor = None
    quant_scale_ckr: torch.Tensor = None
    smooth_scales_cq: torch.Tensor = None


@dataclass
class RopeTileShapeConfig:
    two_dim: List[int] = field(default_factory=list)
    three_dim: List[int] = field(default_factory=list)
    four_dim: List[int] = field(default_factory=list)


_CACHE_MODES = {"PA_BSND": 0}

_SCALARS = ("epsilon_cq", "epsilon_ckv", "cache_mode", "tile_config", "rope_cfg")


def _run(tensors, epsilon_cq, epsilon_ckv, cache_mode):
    if cache_mode not in _CACHE_MODES:
        raise ValueError(f"unsupported cache_mode {cache_mode!r}: only 'PA_BSND' is built")
    launch("mla_prolog_quant", list(tensors),
           MlaPrologParams(float(epsilon_cq), float(epsilon_ckv), _CACHE_MODES[cache_mode]))


@operator(21, _SCALARS)
def mla_prolog_quant_d(*tensors, epsilon_cq, epsilon_ckv, cache_mode, tile_config, rope_cfg):
    """Decode entry.  tensors: token_x, w_dq, w_uq_qr, dequant_scale, w_uk, w_dkv_kr, gamma_cq, gamma_ckv, cos, sin,
    cache_index, kv_cache, kr_cache, k_scale_cache, then the outputs q_norm_out, q_norm_scale_out, query_nope_out,
    query_rope_out, kv_cache_out, kr_cache_out, k_scale_cache_out (the three cache outputs are the cache inputs
    themselves, updated in place at cache_index).  Returns None."""
    _run(tensors, epsilon_cq, epsilon_ckv, cache_mode)


@operator(21, _SCALARS)
def mla_prolog_quant_p(*tensors, epsilon_cq, epsilon_ckv, cache_mode, tile_config, rope_cfg):
    """Prefill entry: same arguments and results as mla_prolog_quant_d (the reference's two entries differ in Ascend
    pass options only)."""
    _run(tensors, epsilon_cq, epsilon_ckv, cache_mode)
