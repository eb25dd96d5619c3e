"""Paged row gather: the rows of a paged KV cache that a list of logical token indices selects.

Same names, argument order and result as the reference's python/pypto/experimental/gather.py:18-84
(``gather_in_ub`` :27-84, ``gather_in_l1`` :18-24); the arithmetic is the interpreter's
(framework/src/interface/interpreter/calculator/calc_torch.cpp:1870-1981):

    out[j, :] = src[block_table[0, idx[0, j] // block_size] * block_size + idx[0, j] % block_size, :]

The device code is the gfx950 HIP kernel behind ``pto_paged_gather_launch``.  In the reference these are tile
operations that return a new tensor (in the unified buffer / L1); here the result is a new tensor in device memory,
written asynchronously on the current stream.
"""
import torch

from .._runtime import PagedGatherParams, launch
from ..error import FeError, PyptoError

_INDEX_DTYPES = (torch.int32, torch.int64)


def _wrap(name, e):
    err = FeError(type(e)(f"Failed to call operator '{name}'.\n{e}"))
    return err.with_traceback(e.__traceback__)


def paged_gather(src, indices, block_table, block_size, size=None, out=None, check=False):
    """Batched form: ``indices [b, k]`` row i is resolved through ``block_table [b, nblk]`` row i; returns
    ``[b * k, size]`` (``size`` defaults to every column of ``src``).

    An entry the reference's interpreter would reject (calc_torch.cpp:1916-1950: index outside the page table,
    negative page, row outside ``src``) gives a row of zeros.  ``check=True`` waits for the launch and raises
    IndexError (wrapped in FeError) if there was such an entry, which is the interpreter's behaviour."""
    try:
        if src.dim() != 2:
            raise ValueError("src must be [token_num, hidden_size]")
        if indices.dim() != 2 or block_table.dim() != 2:
            raise ValueError("indices and block_table must be 2-D")
        if indices.dtype not in _INDEX_DTYPES or block_table.dtype not in _INDEX_DTYPES:
            raise ValueError("indices and block_table must be int32 or int64")
        if not isinstance(block_size, int) or block_size <= 0:
            raise ValueError("block_size must be a positive int")
        width = src.shape[1] if size is None else int(size)
        if width > src.shape[1] or width < 0:
            raise ValueError(f"size ({width}) exceeds the source row width ({src.shape[1]})")
        rows = indices.shape[0] * indices.shape[1]
        if out is None:
            out = torch.empty((rows, width), dtype=src.dtype, device=src.device)
        if width == 0:
            return out
        tensors = [src, indices, block_table, out]
        status = None
        if check:
            status = torch.zeros(1, dtype=torch.int32, device=src.device)
            tensors.append(status)
        launch("paged_gather", tensors, PagedGatherParams(block_size, width))
        if check:
            bad = int(status.item())
            if bad:
                raise IndexError(f"{bad} of {rows} indices address no row of src through the page table")
        return out
    except PyptoError:
        raise
    except Exception as e:  # noqa: BLE001 - everything is re-raised under the boundary's error type
        raise _wrap("paged_gather", e) from None


def gather_in_ub(param, indices, block_table, block_size, axis, check=False):
    """``param [token_num, hidden]``, ``indices [1, k]``, ``block_table [1, nblk]``, ``axis`` -2 (the token axis, the
    only one the reference supports: gather.py:51-53, calc_torch.cpp:1879-1882) -> ``[k, hidden]``."""
    try:
        if param.dim() != 2:
            raise ValueError("param must be [token_num, hidden_size]")
        if axis not in (-2, 0):
            raise ValueError("only axis -2 is supported")
        if indices.dim() != 2 or indices.shape[0] != 1:
            raise ValueError("indices must be [1, k]")
        if block_table.dim() != 2 or block_table.shape[0] != 1:
            raise ValueError("block_table must be [1, block_table_size]")
    except Exception as e:  # noqa: BLE001
        raise _wrap("gather_in_ub", e) from None
    return paged_gather(param, indices, block_table, block_size, check=check)


def gather_in_l1(src, indices, block_table, block_size, size, is_b_matrix=False, is_trans=False, check=False):
    """As ``gather_in_ub`` for the first ``size`` columns of each row -> ``[k, size]``
    (framework/src/interface/operation/operation_impl.cpp:1702-1724).  ``is_b_matrix`` and ``is_trans`` say in
    which L1 layout the Ascend matrix unit wants the rows; the rows themselves are the same, so both are ignored."""
    try:
        if indices.dim() != 2 or indices.shape[0] != 1:
            raise ValueError("indices must be [1, k]")
        if block_table.dim() != 2 or block_table.shape[0] != 1:
            raise ValueError("block_table must be [1, block_table_size]")
        if src.dim() == 2 and size > src.shape[1]:
            raise ValueError(f"size ({size}) exceeds the source row width ({src.shape[1]})")
    except Exception as e:  # noqa: BLE001
        raise _wrap("gather_in_l1", e) from None
    return paged_gather(src, indices, block_table, block_size, size=size, check=check)
