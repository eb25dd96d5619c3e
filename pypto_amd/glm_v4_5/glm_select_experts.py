"""Grouped top-k expert selection of the GLM-4.5 router.

Same entry point, argument order and semantics as the reference's models/glm_v4_5/glm_select_experts.py
(``select_experts`` :316-364, ``check_args`` :36-57); the device code is the gfx950 HIP kernel behind
``pto_select_experts_launch``.  Two optional keyword arguments extend the reference signature with the knobs of
its generalised gating golden (python/tests/ut/interpreter/_ops/moe_gating_topk.py:272,285).
"""
import torch

from .._runtime import SelectExpertsParams, launch
from ..error import FeError, PyptoError


def check_args(router_logits, top_k, renormalize, topk_group, num_expert_group, e_score_correction_bias):
    """The reference's argument assertions (glm_select_experts.py:36-57), widened to the dtypes and expert counts the
    kernel takes: logits fp32 (reference) or bf16, bias bf16 (reference) or fp32, up to 256 experts."""
    assert router_logits.dim() == 2
    assert 1 <= router_logits.shape[1] <= 256
    assert router_logits.dtype in (torch.float32, torch.bfloat16)
    assert e_score_correction_bias.dim() == 1
    assert e_score_correction_bias.shape[0] == router_logits.shape[1]
    assert e_score_correction_bias.dtype in (torch.bfloat16, torch.float32)
    assert isinstance(top_k, int)
    assert isinstance(renormalize, bool)
    assert isinstance(topk_group, int)
    assert isinstance(num_expert_group, int)


def select_experts(router_logits, top_k, renormalize, topk_group, num_expert_group, e_score_correction_bias,
                   topk_weights, topk_ids, routed_scaling_factor=1.0, fill_neg_inf=False):
    """topk_ids[t] = the top_k experts of token t by sigmoid(logit) + bias among the experts of its topk_group best
    groups (a group's score is its largest biased score), in descending order, equal scores by ascending id;
    topk_weights[t] = their un-biased sigmoid scores, divided by their sum if ``renormalize``, times
    ``routed_scaling_factor``.  Experts outside the chosen groups compete with a score of 0.0 (the reference kernel,
    glm_select_experts.py:169) or of -inf (``fill_neg_inf``).  Outputs are written in place; returns None."""
    check_args(router_logits, top_k, renormalize, topk_group, num_expert_group, e_score_correction_bias)
    try:
        params = SelectExpertsParams(int(top_k), int(bool(renormalize)), int(topk_group), int(num_expert_group),
                                     float(routed_scaling_factor), int(bool(fill_neg_inf)))
        launch("select_experts", [router_logits, e_score_correction_bias, topk_weights, topk_ids], params)
    except PyptoError:
        raise
    except Exception as e:  # noqa: BLE001 - everything is re-raised under the boundary's error type
        err = FeError(type(e)(f"Failed to call JIT function 'select_experts_kernel'.\n{e}"))
        raise err.with_traceback(e.__traceback__) from None
    return None
