"""Host side of the operator boundary: torch tensors -> C ABI of libpypto_amd.so.

Plays the role of the reference's call path ``JitCallableWrapper.__call__`` ->
``LaunchKernelTorch`` (python/pypto/frontend/parser/entry.py:296-365,518-583,638-662 and
python/src/bindings/runtime.cpp:625-723): split positional/keyword arguments into tensors and
scalars, check that every tensor is a contiguous torch.Tensor on one device, allocate the workspace
through the torch allocator and launch asynchronously on the caller's current stream.  PyTorch is
used for device memory and streams only; all compute is in the HIP library.
"""
import ctypes
import functools
import os
import struct
import threading
import weakref

import torch

from .error import FeError, PyptoError, PyptoRtError

# PYPTO_AMD_LIBRARY names another build of the library (e.g. the host-sanitizer build of pypto_amd.build)
_LIB_PATH = os.environ.get("PYPTO_AMD_LIBRARY") or os.path.join(os.path.dirname(os.path.abspath(__file__)), "libpypto_amd.so")
_lib = None
_lib_lock = threading.Lock()


class TensorDesc(ctypes.Structure):
    _fields_ = [("addr", ctypes.c_void_p), ("dataType", ctypes.c_int32), ("rank", ctypes.c_int32),
                ("shape", ctypes.c_int64 * 8)]


class SfaParams(ctypes.Structure):
    _fields_ = [("nq", ctypes.c_int32), ("n_kv", ctypes.c_int32), ("softmax_scale", ctypes.c_float),
                ("topk", ctypes.c_int32), ("block_size", ctypes.c_int32),
                ("max_blocknum_perbatch", ctypes.c_int32), ("kv_splits", ctypes.c_int32)]


class IndexerParams(ctypes.Structure):
    _fields_ = [("selected_count", ctypes.c_int32)]


class SelectExpertsParams(ctypes.Structure):
    _fields_ = [("top_k", ctypes.c_int32), ("renormalize", ctypes.c_int32), ("topk_group", ctypes.c_int32),
                ("num_expert_group", ctypes.c_int32), ("routed_scaling_factor", ctypes.c_float),
                ("fill_neg_inf", ctypes.c_int32)]


# framework/include/tilefwk/data_type.h:33-65
_DTYPE_CODE = {torch.int8: 1, torch.int32: 3, torch.int64: 4, torch.float16: 6, torch.float32: 7, torch.bfloat16: 8}

class GqaParams(ctypes.Structure):
    _fields_ = [("softmax_scale", ctypes.c_float), ("kv_chunk", ctypes.c_int32)]


class IndexerPrologParams(ctypes.Structure):
    _fields_ = [("eps", ctypes.c_float)]


class MlaPrologParams(ctypes.Structure):
    _fields_ = [("epsilon_cq", ctypes.c_float), ("epsilon_ckv", ctypes.c_float), ("cache_mode", ctypes.c_int32)]


class MlaIndexerPrologParams(ctypes.Structure):
    _fields_ = [("epsilon_cq", ctypes.c_float), ("epsilon_ckv", ctypes.c_float), ("cache_mode", ctypes.c_int32),
                ("indexer_eps", ctypes.c_float)]


class AttentionPreQuantParams(ctypes.Structure):
    _fields_ = [("eps", ctypes.c_float)]


class TopkParams(ctypes.Structure):
    _fields_ = [("k", ctypes.c_int32), ("largest", ctypes.c_int32)]


class PagedGatherParams(ctypes.Structure):
    _fields_ = [("block_size", ctypes.c_int32), ("size", ctypes.c_int32)]


_OPS = {
    "sfa_quant": SfaParams,
    "sfa_antiquant": SfaParams,
    "lightning_indexer": IndexerParams,
    "select_experts": SelectExpertsParams,
    "gqa_decode": GqaParams,
    "indexer_prolog": IndexerPrologParams,
    "mla_prolog_quant": MlaPrologParams,
    "mla_indexer_prolog_quant": MlaIndexerPrologParams,
    "attention_pre_quant": AttentionPreQuantParams,
    "paged_gather": PagedGatherParams,
    "topk": TopkParams,
}

# C status -> Python exception type wrapped by FeError
_STATUS_EXC = {-1: RuntimeError, -2: ValueError, -3: ValueError, -4: ValueError, -5: RuntimeError, -6: RuntimeError,
               -7: RuntimeError, -8: ValueError}


def library_path():
    return _LIB_PATH


def load_library():
    """Load libpypto_amd.so (built in-tree by ``python -m pypto_amd.build``).  There is no fallback:
    without the library every operator call fails."""
    global _lib
    if _lib is not None:
        return _lib
    with _lib_lock:
        if _lib is not None:
            return _lib
        if not os.path.exists(_LIB_PATH):
            raise PyptoRtError(RuntimeError(
                f"{_LIB_PATH} is missing: build it with `python -m pypto_amd.build` (hipcc, gfx950)"))
        lib = ctypes.CDLL(_LIB_PATH)
        for op, ptype in _OPS.items():
            ws = getattr(lib, f"pto_{op}_workspace")
            ws.restype = ctypes.c_uint64
            ws.argtypes = [ctypes.POINTER(TensorDesc), ctypes.c_uint32, ctypes.POINTER(ptype)]
            ln = getattr(lib, f"pto_{op}_launch")
            ln.restype = ctypes.c_int
            ln.argtypes = [ctypes.POINTER(TensorDesc), ctypes.c_uint32, ctypes.POINTER(ptype), ctypes.c_void_p,
                           ctypes.c_uint64, ctypes.c_void_p, ctypes.c_int]
        lib.pto_last_error.restype = ctypes.c_char_p
        lib.pto_last_error.argtypes = []
        lib.pto_abi_version.restype = ctypes.c_int
        _lib = lib
    return _lib


_DESC = struct.Struct("Pii8q")          # PtoTensorDesc: addr, dataType, rank, shape[8]
assert _DESC.size == ctypes.sizeof(TensorDesc)
_PAD = tuple((0,) * (8 - r) for r in range(9))


def describe(tensors):
    """PtoTensorDesc array of the tensors (no checks beyond dtype and rank)."""
    n = len(tensors)
    buf = bytearray(_DESC.size * n)
    off = 0
    for t in tensors:
        code = _DTYPE_CODE.get(t.dtype)
        if code is None:
            raise ValueError(f"unsupported tensor dtype {t.dtype}")
        shape = t.shape
        r = len(shape)
        if r > 8:
            raise ValueError("tensors of more than 8 dimensions are not supported")
        _DESC.pack_into(buf, off, t.data_ptr() if t.numel() else 0, code, r, *shape, *_PAD[r])
        off += _DESC.size
    return (TensorDesc * n).from_buffer(buf)


def _check_and_describe(tensors):
    """The checks of the reference's binding (every operand a dense torch.Tensor, all on one HIP device) and the
    descriptor array, in one pass over the tensors: this is the host's cost of a call, and it shows for the operators
    whose kernels take a few tens of microseconds."""
    n = len(tensors)
    buf = bytearray(_DESC.size * n)
    off = 0
    dev = None
    for idx, t in enumerate(tensors):
        if type(t) is not torch.Tensor:
            if not isinstance(t, torch.Tensor):
                raise FeError(RuntimeError(f"Input {idx + 1} (index {idx}) must be a torch.Tensor, got {t.__class__}"))
            if type(t).__name__ == "DTensor":
                raise FeError(RuntimeError(f"Input {idx + 1} (index {idx}) must not be a DTensor, got {t.__class__}"))
        if not t.is_contiguous():
            raise FeError(RuntimeError("not all tensors are contiguous"))
        d = t.device
        if dev is None:
            dev = d
        elif d != dev:
            raise FeError(RuntimeError(f"all tensors must be on the same device, got {dev} and {d}"))
        code = _DTYPE_CODE.get(t.dtype)
        if code is None:
            raise ValueError(f"unsupported tensor dtype {t.dtype}")
        shape = t.shape
        r = len(shape)
        if r > 8:
            raise ValueError("tensors of more than 8 dimensions are not supported")
        _DESC.pack_into(buf, off, t.data_ptr() if t.numel() else 0, code, r, *shape, *_PAD[r])
        off += _DESC.size
    if dev.type != "cuda":
        raise FeError(RuntimeError(f"tensors must be on a HIP device (torch device type 'cuda'), got {dev}"))
    descs = (TensorDesc * n).from_buffer(buf)
    descs._buf = buf  # (the planned path rewrites addresses in place)
    return dev, descs


_fns = {}


def _entry_points(op):
    fns = _fns.get(op)
    if fns is None:
        lib = load_library()
        fns = _fns[op] = (getattr(lib, f"pto_{op}_workspace"), getattr(lib, f"pto_{op}_launch"))
    return fns


def _launch_on_current_device(dev, launch_fn, descs, n, params_ref, ws_bytes):
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev) if ws_bytes else None
    return launch_fn(descs, n, params_ref, ws.data_ptr() if ws is not None else None, ws_bytes,
                     torch.cuda.current_stream(dev).cuda_stream, 0)


class _Plan:
    """What a call leaves behind for the next call of the same operator on the same thread: the checked descriptor
    array and the workspace size.  The reference keeps a compiled kernel module per (operator, argument shapes) and
    skips compilation on a hit (python/pypto/frontend/parser/entry.py:613-636, python/src/bindings/runtime.cpp:430-523);
    what there is to skip here is the validation of the tensor list and the workspace query."""
    __slots__ = ("refs", "shapes", "ptrs", "buf", "descs", "n", "params", "params_ref", "ws_bytes", "dev", "current")


_tls = threading.local()
_PTR = struct.Struct("P")


def _check_one(idx, t, dev):
    """The per-tensor checks of _check_and_describe for one operand of a planned call; returns its dtype code."""
    if type(t) is not torch.Tensor:
        if not isinstance(t, torch.Tensor):
            raise FeError(RuntimeError(f"Input {idx + 1} (index {idx}) must be a torch.Tensor, got {t.__class__}"))
        if type(t).__name__ == "DTensor":
            raise FeError(RuntimeError(f"Input {idx + 1} (index {idx}) must not be a DTensor, got {t.__class__}"))
    if not t.is_contiguous():
        raise FeError(RuntimeError("not all tensors are contiguous"))
    if t.device != dev:
        raise FeError(RuntimeError(f"all tensors must be on the same device, got {dev} and {t.device}"))
    code = _DTYPE_CODE.get(t.dtype)
    if code is None:
        raise ValueError(f"unsupported tensor dtype {t.dtype}")
    if len(t.shape) > 8:
        raise ValueError("tensors of more than 8 dimensions are not supported")
    return code


def _refresh(plan, tensors, params, ws_fn):
    """Brings the plan up to date with this call, operand by operand: an operand that is the very object of the planned
    call, unchanged in shape and layout, only has its address looked at (storage can be reallocated under a live
    tensor); any other operand - another layer's weights, a new activation - is checked and described afresh.  The
    workspace is sized again only if a shape or the scalar parameters changed.  False: plan from scratch."""
    if plan.n != len(tensors):
        return False
    resize = False
    pb = bytes(params)
    if pb != plan.params:
        plan.params = pb
        plan.params_ref = ctypes.byref(params.__class__.from_buffer_copy(pb))
        resize = True
    refs, shapes, ptrs, buf, dev = plan.refs, plan.shapes, plan.ptrs, plan.buf, plan.dev
    i = 0
    for t in tensors:
        if refs[i]() is t and t.shape == shapes[i] and t.is_contiguous():
            p = t.data_ptr() if ptrs[i] else 0  # (an empty tensor's descriptor carries a null address)
            if p != ptrs[i]:
                _PTR.pack_into(buf, i * _DESC.size, p)
                ptrs[i] = p
        else:
            code = _check_one(i, t, dev)
            shape = t.shape
            r = len(shape)
            p = t.data_ptr() if t.numel() else 0
            _DESC.pack_into(buf, i * _DESC.size, p, code, r, *shape, *_PAD[r])
            resize = resize or shape != shapes[i]
            refs[i], shapes[i], ptrs[i] = weakref.ref(t), shape, p
        i += 1
    if resize:
        plan.ws_bytes = ws_fn(plan.descs, plan.n, plan.params_ref)
    return True


def launch(op, tensors, params):
    """Validate, size the workspace, launch on the current stream of the tensors' device.  A repeated call of an
    operator takes the planned path (_refresh)."""
    plans = getattr(_tls, "plans", None)
    if plans is None:
        plans = _tls.plans = {}
    ws_fn, launch_fn = _entry_points(op)
    plan = plans.get(op)
    try:
        hit = plan is not None and _refresh(plan, tensors, params, ws_fn)
    except Exception:
        plans.pop(op, None)  # the buffer may be half rewritten
        raise
    if not hit:
        dev, descs = _check_and_describe(tensors)
        plan = _Plan()
        plan.n = len(tensors)
        plan.refs = [weakref.ref(t) for t in tensors]
        plan.shapes = [t.shape for t in tensors]
        plan.ptrs = [t.data_ptr() if t.numel() else 0 for t in tensors]
        plan.descs = descs
        plan.buf = descs._buf
        plan.params = bytes(params)
        plan.params_ref = ctypes.byref(params.__class__.from_buffer_copy(plan.params))
        plan.ws_bytes = ws_fn(descs, plan.n, plan.params_ref)
        plan.dev = dev
        plan.current = dev.index is None
        plans[op] = plan
    dev = plan.dev
    if plan.current or dev.index == torch.cuda.current_device():
        rc = _launch_on_current_device(dev, launch_fn, plan.descs, plan.n, plan.params_ref, plan.ws_bytes)
    else:
        with torch.cuda.device(dev):
            rc = _launch_on_current_device(dev, launch_fn, plan.descs, plan.n, plan.params_ref, plan.ws_bytes)
    if rc != 0:
        plans.pop(op, None)
        msg = _lib.pto_last_error().decode()
        raise _STATUS_EXC.get(rc, RuntimeError)(msg)


def operator(n_tensors, scalar_names):
    """Call convention of a jit-compiled reference operator: the first ``n_tensors`` positional
    arguments are tensors (outputs included, caller-allocated), the rest are non-tensor arguments,
    positional or by keyword; returns None; every failure surfaces as FeError
    (python/pypto/frontend/parser/entry.py:296-322,518-583)."""

    def deco(fn):
        @functools.wraps(fn)
        def wrapper(*args, **kwargs):
            try:
                if len(args) < n_tensors:
                    raise RuntimeError(f"{fn.__name__} takes {n_tensors} tensors, got {len(args)} positional arguments")
                tensors = list(args[:n_tensors])
                rest = list(args[n_tensors:])
                if len(rest) > len(scalar_names):
                    raise RuntimeError(f"{fn.__name__} takes {len(scalar_names)} non-tensor arguments, got {len(rest)}")
                scalars = dict(zip(scalar_names, rest))
                for k, v in kwargs.items():
                    if k not in scalar_names:
                        raise TypeError(f"{fn.__name__} got an unexpected keyword argument '{k}'")
                    scalars[k] = v
                missing = [k for k in scalar_names if k not in scalars]
                if missing:
                    raise TypeError(f"{fn.__name__} missing non-tensor arguments: {', '.join(missing)}")
                fn(*tensors, **scalars)
            except PyptoError:
                raise
            except Exception as e:  # noqa: BLE001 - everything is re-raised under the boundary's error type
                err = FeError(type(e)(f"Failed to call JIT function '{fn.__name__}'.\n{e}"))
                raise err.with_traceback(e.__traceback__) from None
            return None

        return wrapper

    return deco
