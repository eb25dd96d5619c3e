"""Top-k ordering rule (CPU oracle, test infrastructure).

The reference defines top-k as ``torch.topk(sorted=True)``
(framework/tests/st/operation/python/vector_operator_golden.py:2247-2259) and
its interpreter then fixes the order of equal values: smaller index first
(framework/src/interface/interpreter/calculator/calc_torch.cpp:2481-2494,2734-2749).
"""
import numpy as np
import torch


def topk_sorted_stable(row, k, largest=True):
    """k extreme elements of a 1-D tensor, best first, ties by ascending index.

    Returns (values, int32 indices).
    """
    x = torch.as_tensor(row).reshape(-1)
    order = torch.sort(x, descending=largest, stable=True).indices[:k]
    return x[order], order.to(torch.int32)


def topk_rows(x2d, k, largest=True):
    vals, idxs = [], []
    for r in range(x2d.shape[0]):
        v, i = topk_sorted_stable(x2d[r], k, largest)
        vals.append(v)
        idxs.append(i)
    return torch.stack(vals), torch.stack(idxs)
