"""Mirror of the reference's ``pypto.topk`` (python/pypto/op/comparison.py:302-344) on the HIP library.

``topk(input, k, dim=None, largest=True)`` returns ``(values, indices)``: the k largest (smallest) elements along
``dim`` (the last dimension when not given), best first, indices int32; equal values come in ascending index order, the
order the reference's interpreter fixes (framework/src/interface/interpreter/calculator/calc_torch.cpp:2481-2494).
The reference builds a graph node and returns its output tensors; here the outputs are allocated with torch and the
kernel is launched on the current stream.  ``algo`` (MERGE_SORT / RADIX_SELECT) selects between Ascend code paths and is
accepted and ignored.
"""
import torch

from .. import _runtime
from ..error import FeError


def topk(input, k, dim=None, largest=True, algo=None):  # noqa: A002 - the reference's parameter name
    try:
        if not isinstance(input, torch.Tensor):
            raise TypeError(f"topk: input must be a torch.Tensor, got {type(input)}")
        if input.dtype != torch.float32:
            raise ValueError(f"topk: input must be float32 (the reference's sort takes fp32 only), got {input.dtype}")
        if input.dim() == 0:
            raise ValueError("topk: input must have at least one dimension")
        d = -1 if dim is None else int(dim)
        if not -input.dim() <= d < input.dim():
            raise ValueError(f"topk: dim {d} out of range for a {input.dim()}-dimensional tensor")
        x = input.movedim(d, -1)
        lead, n = x.shape[:-1], x.shape[-1]
        x2 = x.reshape(-1, n).contiguous()
        k = int(k)
        values = torch.empty((x2.shape[0], k), dtype=torch.float32, device=x2.device)
        indices = torch.empty((x2.shape[0], k), dtype=torch.int32, device=x2.device)
        _runtime.launch("topk", [x2, values, indices], _runtime.TopkParams(k, 1 if largest else 0))
        return (values.reshape(*lead, k).movedim(-1, d), indices.reshape(*lead, k).movedim(-1, d))
    except FeError:
        raise
    except Exception as e:  # noqa: BLE001 - the boundary's error type
        raise FeError(type(e)(f"Failed to call JIT function 'topk'.\n{e}")).with_traceback(e.__traceback__) from None
