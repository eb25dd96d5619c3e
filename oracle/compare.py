"""Tolerance comparators of the reference's operator tests (CPU oracle, test infrastructure).

``compare``           models/deepseek_v32_exp/utils/compare.py:16-125
``topk_idx_compare``  models/deepseek_v32_exp/deepseekv32_lightning_indexer_quant.py:266-307
"""
import torch


def count_violations(t, t_ref, atol, rtol):
    d = (t.to(torch.float64) - t_ref.to(torch.float64)).abs()
    return int((d > atol + rtol * t_ref.to(torch.float64).abs()).sum())


def compare(t, t_ref, name, atol, rtol, max_error_ratio=0.005):
    """Fail on NaN/Inf, on shape/dtype/device mismatch, or when more than
    round(max_error_ratio * numel) elements violate |t-ref| <= atol + rtol*|ref|."""
    assert not torch.isnan(t).any(), f"{name}: NaN in result"
    assert not torch.isinf(t).any(), f"{name}: Inf in result"
    assert t.shape == t_ref.shape, f"{name}: shape {tuple(t.shape)} vs {tuple(t_ref.shape)}"
    assert t.dtype == t_ref.dtype, f"{name}: dtype {t.dtype} vs {t_ref.dtype}"
    assert t.device == t_ref.device, f"{name}: device {t.device} vs {t_ref.device}"
    limit = round(max_error_ratio * t_ref.numel())
    diff = (t - t_ref).abs()
    bad = int((diff > atol + rtol * t_ref.abs()).sum())
    assert bad <= limit, f"compare fail: {name}, max diff {float(diff.max()):.8f}, error_count {bad}, threshold {limit}"
    return bad


def topk_idx_compare(t, t_ref, name, ratio=5e-4, group=2048):
    """Per group of ``group`` output slots: gather the positions that differ,
    then count reference ids that are absent from the produced ids of that
    group; at most int(group * ratio) may be missing."""
    a = t.reshape(-1).tolist()
    e = t_ref.reshape(-1).tolist()
    assert len(a) == len(e), f"{name}: length mismatch"
    allowed = int(group * ratio)
    worst = 0
    for g0 in range(0, len(e), group):
        exp_bad, act_bad = [], set()
        for x, y in zip(a[g0:g0 + group], e[g0:g0 + group]):
            if x != y:
                exp_bad.append(y)
                act_bad.add(x)
        missing = sum(1 for y in exp_bad if y not in act_bad)
        worst = max(worst, missing)
        assert missing <= allowed, f"compare fail: {name}, group {g0 // group}: {missing} ids missing (allowed {allowed})"
    return worst
