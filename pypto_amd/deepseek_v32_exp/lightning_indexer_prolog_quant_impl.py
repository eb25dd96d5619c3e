"""Lightning-indexer prolog: the producer of the indexer's query, per-head weights and paged int8 index-key cache.

Same entry point, dataclasses, argument order and semantics as the reference module
models/deepseek_v32_exp/lightning_indexer_prolog_quant_impl.py (``IndexerPrologQuantInput`` :63-80,
``IndexerPrologQuantOutput`` :83-89, ``IndexerPrologQuantAttr`` :92-96, ``IndexerPrologQuantConfigs`` :99-112,
``lightning_indexer_prolog_quant`` :203-243); the device code is the gfx950 HIP kernels behind
``pto_indexer_prolog_launch``.  The weights are taken in plain row-major layout (the reference casts them to the
Ascend NZ tiling, a device format, before the call).
"""
from dataclasses import dataclass, field
from typing import List

import torch

from .._runtime import IndexerPrologParams, launch, operator


@dataclass
class IndexerPrologQuantInput:
    x: torch.Tensor  # BF16, (t, h)
    q_norm: torch.Tensor  # INT8, (t, q_lora_rank)
    q_norm_scale: torch.Tensor  # FP32, (t, 1)
    w_qb: torch.Tensor  # INT8, (q_lora_rank, head_num * head_dim)
    w_qb_scale: torch.Tensor  # FP32, (head_num * head_dim, 1)
    wk: torch.Tensor  # BF16, (h, head_dim)
    w_proj: torch.Tensor  # BF16, (h, head_num)
    ln_gamma_k: torch.Tensor  # BF16, (head_dim,)
    ln_beta_k: torch.Tensor  # BF16, (head_dim,)
    cos_idx_rope: torch.Tensor  # BF16, (t, rope_head_dim)
    sin_idx_rope: torch.Tensor  # BF16, (t, rope_head_dim)
    hadamard_q: torch.Tensor  # BF16, (head_dim, head_dim)
    hadamard_k: torch.Tensor  # BF16, (head_dim, head_dim)
    k_cache: torch.Tensor  # INT8, (block_num, block_size, n_kv, head_dim)
    k_cache_scale: torch.Tensor  # FP16, (block_num, block_size, n_kv, 1)
    k_cache_index: torch.Tensor  # INT64, (t,)


@dataclass
class IndexerPrologQuantOutput:
    q_int8: torch.Tensor
    q_scale: torch.Tensor
    k_int8: torch.Tensor
    k_scale: torch.Tensor
    weights: torch.Tensor


@dataclass
class IndexerPrologQuantAttr:
    eps: float = 1e-6
    layerout_query: str = "TND"
    layerout_key: str = "PA_BSND"


@dataclass
class IndexerPrologQuantConfigs:
    """Ascend tiling knobs of the reference operator; accepted for call compatibility and ignored."""
    q_linear: List[int] = field(default_factory=list)
    q_hd: List[int] = field(default_factory=list)
    k_linear: List[int] = field(default_factory=list)
    w_linear: List[int] = field(default_factory=list)
    unroll_list: List[int] = field(default_factory=list)
    cube_l1_reuse_setting: dict = field(default_factory=dict)
    block_size: int = 128
    t_sub_tile: int = 1
    chunk_size: int = 2
    vec_nbuffer_setting: dict = field(default_factory=dict)


@operator(21, ("configs", "attrs"))
def lightning_indexer_prolog_quant(*tensors, configs, attrs):
    """tensors: the 16 fields of IndexerPrologQuantInput followed by the 5 of IndexerPrologQuantOutput; k_int8 and
    k_scale are the k_cache and k_cache_scale buffers themselves (updated in place at k_cache_index).  Writes q_int8,
    q_scale, the cache rows and weights; returns None."""
    if attrs.layerout_query != "TND" or attrs.layerout_key != "PA_BSND":
        raise ValueError(f"unsupported layouts {attrs.layerout_query!r} / {attrs.layerout_key!r}")
    launch("indexer_prolog", list(tensors), IndexerPrologParams(float(attrs.eps)))
