"""Shared helpers for the GPU parity tests: run an oracle-generated case through the operator boundary."""
import math

import torch

from oracle import indexer as oi
from oracle import sfa as osfa
from pypto_amd.deepseek_v32_exp import lightning_indexer_quant_impl as li_impl
from pypto_amd.deepseek_v32_exp import sparse_attention_antiquant_impl as aq_impl
from pypto_amd.deepseek_v32_exp import sparse_flash_attention_quant_impl as sfa_impl


def run_sfa(case, dev, entry="d", packed=False):
    b, s1, nq, topk = case["b"], case["s1"], case["nq"], case["topk"]
    q = case["q"]
    qn = q[..., :512].reshape(b * s1 * nq, 512).contiguous().to(dev)
    qr = q[..., 512:].reshape(b * s1 * nq, 64).contiguous().to(dev)
    tk = case["topk_indices"].to(dev)
    bt = case["block_table"].to(dev)
    act = torch.tensor(case["act_seq"], dtype=torch.int32, device=dev)
    max_blocks = bt.shape[1]
    scale = case["softmax_scale"]
    if packed:
        rows = osfa.pack_cache_rows(case["kn"], case["kr"], case["kn_scales"]).to(dev)
        out = torch.zeros((b * s1 * nq, 512), dtype=torch.bfloat16, device=dev)
        fn = {"d": aq_impl.sparse_attention_antiquant_d, "p": aq_impl.sparse_attention_antiquant_p,
              "d_950": aq_impl.sparse_attention_antiquant_d_950}[entry]
        fn(qn, qr, rows, tk, bt, act, out, nq, 1, scale, topk, case["block_size"], max_blocks,
           aq_impl.SaTileShapeConfig())
        torch.cuda.synchronize()
        return out.reshape(b, s1, nq, 512).cpu()
    out = torch.zeros((b, s1, nq, 512), dtype=torch.bfloat16, device=dev)
    fn = {"d": sfa_impl.sparse_flash_attention_quant_d, "p": sfa_impl.sparse_flash_attention_quant_p,
          "d_950": sfa_impl.sparse_flash_attention_quant_d_950}[entry]
    fn(qn, qr, case["kn"].to(dev), case["kr"].to(dev), case["kn_scales"].to(dev), tk, bt, act, out, nq, 1, scale,
       topk, case["block_size"], max_blocks, sfa_impl.SaTileShapeConfig())
    torch.cuda.synchronize()
    return out.cpu()


def sfa_golden(case, flash=False, s2_tile=512):
    args = (case["q"], case["kn"], case["kr"], case["kn_scales"], case["topk_indices"], case["block_table"],
            case["act_seq"], case["block_size"], case["softmax_scale"], case["topk"])
    return osfa.attention_flash(*args, s2_tile=s2_tile) if flash else osfa.attention_no_flash(*args)


def run_indexer(case, dev):
    t = case["b"] * case["s1"]
    out = torch.zeros((t, 1, case["selected_count"]), dtype=torch.int32, device=dev)
    li_impl.lightning_indexer_decode(
        case["query"].to(dev), case["q_scale"].to(dev), case["key_cache"].to(dev), case["k_scale"].to(dev),
        case["weights"].to(dev), torch.tensor(case["act_seq"], dtype=torch.int32, device=dev),
        case["block_table"].to(dev), out, [128, 64, 32, 16, 8, 4, 1], li_impl.LightningIndexerConfigs(),
        case["selected_count"])
    torch.cuda.synchronize()
    return out.cpu()


def indexer_scores(case, exact=False):
    fn = oi.scores_exact if exact else oi.scores
    return fn(case["query"], case["q_scale"], case["key_cache"], case["k_scale"], case["weights"], case["act_seq"],
              case["block_table"], case["s1"])
