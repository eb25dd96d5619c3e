"""Fused MLA prolog + lightning-indexer prolog: one call that turns hidden states into the attention query, the new rows
of the paged int8 MLA cache, and the indexer's query, weights and new index-cache rows.

Same entry points, argument order and semantics as the reference module
models/deepseek_v32_exp/mla_indexer_prolog_quant_impl.py (``mla_indexer_prolog_quant_p`` :320-477,
``mla_indexer_prolog_quant_d`` :479-634): the MLA prolog's q_norm / q_norm_scale stay internal and feed the indexer
prolog; token_x, cos, sin and cache_index are shared.  The device code is the gfx950 HIP kernels of the two operators,
launched back to back on the caller's stream behind ``pto_mla_indexer_prolog_quant_launch``.
"""
from .._runtime import MlaIndexerPrologParams, launch, operator
from .lightning_indexer_prolog_quant_impl import IndexerPrologQuantAttr, IndexerPrologQuantConfigs  # noqa: F401
from .mla_prolog_quant_impl import _CACHE_MODES, MlaTileConfig, RopeTileShapeConfig  # noqa: F401

_SCALARS = ("mla_epsilon_cq", "mla_epsilon_ckv", "mla_cache_mode", "mla_tile_config", "ip_attrs", "ip_configs", "rope_cfg")


def _run(tensors, mla_epsilon_cq, mla_epsilon_ckv, mla_cache_mode, ip_attrs):
    if mla_cache_mode not in _CACHE_MODES:
        raise ValueError(f"unsupported mla_cache_mode {mla_cache_mode!r}: only 'PA_BSND' is built")
    if ip_attrs.layerout_query != "TND" or ip_attrs.layerout_key != "PA_BSND":
        raise ValueError(f"unsupported layouts {ip_attrs.layerout_query!r} / {ip_attrs.layerout_key!r}")
    launch("mla_indexer_prolog_quant", list(tensors),
           MlaIndexerPrologParams(float(mla_epsilon_cq), float(mla_epsilon_ckv), _CACHE_MODES[mla_cache_mode],
                                  float(ip_attrs.eps)))


@operator(34, _SCALARS)
def mla_indexer_prolog_quant_d(*tensors, mla_epsilon_cq, mla_epsilon_ckv, mla_cache_mode, mla_tile_config, ip_attrs,
                               ip_configs, rope_cfg):
    """Decode entry.  tensors: token_x, mla_w_dq, mla_w_uq_qr, mla_dequant_scale, mla_w_uk, mla_w_dkv_kr, mla_gamma_cq,
    mla_gamma_ckv, cos, sin, cache_index, mla_kv_cache, mla_kr_cache, mla_k_scale_cache, ip_w_qb_in, ip_w_qb_scale_in,
    ip_wk_in, ip_w_proj_in, ip_ln_gamma_k_in, ip_ln_beta_k_in, ip_hadamard_q_in, ip_hadamard_k_in, ip_k_cache,
    ip_k_cache_scale, then the outputs mla_query_nope_out, mla_query_rope_out, mla_kv_cache_out, mla_kr_cache_out,
    mla_k_scale_cache_out, ip_q_int8_out, ip_q_scale_out, ip_k_int8_out, ip_k_scale_out, ip_weights_out (the cache
    outputs are the cache inputs themselves, updated in place at cache_index).  Returns None."""
    _run(tensors, mla_epsilon_cq, mla_epsilon_ckv, mla_cache_mode, ip_attrs)


@operator(34, _SCALARS)
def mla_indexer_prolog_quant_p(*tensors, mla_epsilon_cq, mla_epsilon_ckv, mla_cache_mode, mla_tile_config, ip_attrs,
                               ip_configs, rope_cfg):
    """Prefill entry: same arguments and results as mla_indexer_prolog_quant_d (the reference's two entries differ in
    Ascend pass options only)."""
    _run(tensors, mla_epsilon_cq, mla_epsilon_ckv, mla_cache_mode, ip_attrs)
