"""Lightning indexer decode: int8 index scores, ReLU, per-head weights, top-k token selection.

Same entry point, argument order and semantics as the reference module
models/deepseek_v32_exp/lightning_indexer_quant_impl.py (``lightning_indexer_decode`` :226-238);
``LightningIndexerConfigs`` is re-declared from
models/deepseek_v32_exp/deepseekv32_lightning_indexer_quant.py:26-43 so callers construct it unchanged.
"""
from dataclasses import dataclass

from .._runtime import IndexerParams, launch, operator

MAX_LI_S1 = 4
MAX_LI_S2 = 128 * 1024


@dataclass
class LightningIndexerConfigs:
    """Ascend tiling knobs; accepted and ignored.  The one semantic field of the reference,
    extend_param = {scale: 1/2048, relu}, is fixed in the kernel."""
    s1_tile: int = 2
    topk_tile: int = 8192


@operator(8, ("unroll_list", "configs", "selected_count"))
def lightning_indexer_decode(idx_query, idx_query_scale, idx_key_cache, idx_key_scale, idx_weight, act_seq_key,
                             block_table, topk_res, unroll_list, configs, selected_count):
    """topk_res[t, 1, selected_count] <- indices of the selected_count best-scoring cached tokens of each
    query token (best first, -1 beyond the token's valid length).  The scales are fp16 as in the reference, or both
    fp32 (per-token scales kept in fp32; then the per-head factor is fp16(idx_query_scale * fp32(idx_weight)) and
    idx_key_scale multiplies the head sum unrounded)."""
    launch("lightning_indexer", [idx_query, idx_query_scale, idx_key_cache, idx_key_scale, idx_weight, act_seq_key,
                                 block_table, topk_res], IndexerParams(int(selected_count)))
