"""CPU restatement of the reference's grouped expert selection (test infrastructure only, never the product path).

Follows the golden written inline in models/glm_v4_5/glm_select_experts.py:274-313 (sigmoid, + bias, group maximum,
top groups, experts of the other groups filled with 0.0, top-k experts, weights gathered from the un-biased sigmoid,
renormalised) and its generalisation python/tests/ut/interpreter/_ops/moe_gating_topk.py:223-287 (groups > 1, experts of
the other groups filled with -inf, stable tie-break, routed scaling factor).  Ordering rule of the device operator
(framework/src/interface/interpreter/calculator/calc_torch.cpp:2481-2494): descending value, equal values in ascending
index order - which is what a stable argsort of the negated values gives.
"""
import torch


def select_experts(router_logits, top_k, renormalize, topk_group, num_expert_group, e_score_correction_bias,
                   routed_scaling_factor=1.0, fill_neg_inf=False):
    """Returns (topk_weights [T, top_k] fp32, topk_ids [T, top_k] int32)."""
    t, ne = router_logits.shape
    s = router_logits.float().sigmoid()                        # glm_select_experts.py:276-277
    x = s + e_score_correction_bias.float().unsqueeze(0)       # :278-279
    if True:  # with one group the mask keeps every expert, as in both references
        g = x.view(t, num_expert_group, ne // num_expert_group).max(dim=-1).values   # :280-281
        order = torch.argsort(-g, dim=-1, stable=True)[:, :topk_group]               # :283 / moe_gating_topk.py:268
        keep = torch.zeros((t, num_expert_group), dtype=torch.bool)
        keep.scatter_(1, order, True)                                                # :284-286
        keep = keep.unsqueeze(-1).expand(t, num_expert_group, ne // num_expert_group).reshape(t, ne)  # :287-289
        fill = float("-inf") if fill_neg_inf else 0.0                                # :291 / moe_gating_topk.py:272
        x = torch.where(keep, x, torch.full_like(x, fill))
    ids = torch.argsort(-x, dim=-1, stable=True)[:, :top_k]                          # :293 / moe_gating_topk.py:276-277
    w = s.gather(1, ids)                                                             # :296
    if renormalize:
        w = w / w.sum(dim=-1, keepdim=True)                                          # :298-299
    w = w * routed_scaling_factor                                                    # moe_gating_topk.py:285
    return w.float(), ids.to(torch.int32)


def biased_scores(router_logits, e_score_correction_bias):
    """The values the selection compares (fp32), for tests that need score gaps."""
    return router_logits.float().sigmoid() + e_score_correction_bias.float().unsqueeze(0)


def make_case(t, ne=160, seed=0, logits_dtype=torch.float32, bias_dtype=torch.bfloat16, dist="normal"):
    """dist "normal": the benchmark's expert-selector configuration (logits N(0,1), bias N(0,0.1));
    dist "uniform": the reference test's inputs (both U[0,1), glm_select_experts.py:262-263)."""
    g = torch.Generator().manual_seed(seed)
    if dist == "uniform":
        logits = torch.rand((t, ne), generator=g)
        bias = torch.rand((ne,), generator=g)
    else:
        logits = torch.randn((t, ne), generator=g)
        bias = 0.1 * torch.randn((ne,), generator=g)
    return logits.to(logits_dtype), bias.to(bias_dtype)
