"""Host side of the operator boundary: torch tensors -> C ABI of libpypto_amd.so.

Plays the role of the reference's call path ``JitCallableWrapper.__call__`` ->
``LaunchKernelTorch`` (python/pypto/frontend/parser/entry.py:296-365,518-583,638-662 and
python/src/bindings/runtime.cpp:625-723): split positional/keyword arguments into tensors and
scalars, check that every tensor is a contiguous torch.Tensor on one device, allocate the workspace
through the torch allocator and launch asynchronously on the caller's current stream.  The checks, the
descriptor list and the launch are C++ (csrc/host_binding.cpp, a pybind11 module over the C ABI);
this file holds the scalar-parameter blocks, the call convention of the operators and a ctypes
binding of the same C ABI for tests and measurement hooks.  PyTorch is used for device memory and
streams only; all compute is in the HIP library.
"""
import ctypes
import functools
import os
import struct
import threading

import torch

from .error import FeError, PyptoError, PyptoRtError

# PYPTO_AMD_LIBRARY names another build of the library (e.g. the host-sanitizer build of pypto_amd.build)
_LIB_PATH = os.environ.get("PYPTO_AMD_LIBRARY") or os.path.join(os.path.dirname(os.path.abspath(__file__)), "libpypto_amd.so")
_lib = None
_lib_lock = threading.RLock()
ABI_VERSION = 2  # include/pypto_amd.h: every launch ends in (workspace, workspace_bytes, hip_stream, sync)


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
        if lib.pto_abi_version() != ABI_VERSION:
            raise PyptoRtError(RuntimeError(
                f"{_LIB_PATH} has ABI version {lib.pto_abi_version()}, this package needs {ABI_VERSION}: rebuild it "
                f"with `python -m pypto_amd.build`"))
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


_host_mod = None


def load_host():
    """The pybind11 layer (pypto_amd/_host.so, built by ``python -m pypto_amd.build``): the product's call path from
    torch tensors to the C ABI.  There is no fallback: without it every operator call fails."""
    global _host_mod
    if _host_mod is not None:
        return _host_mod
    load_library()  # the C ABI library first: a clear message when it is the one that is missing
    with _lib_lock:
        if _host_mod is None:
            try:
                from . import _host
            except ImportError as e:
                raise PyptoRtError(RuntimeError(
                    f"pypto_amd._host is missing or does not load ({e}): build it with `python -m pypto_amd.build`")) from None
            if _host.ABI_VERSION != ABI_VERSION:
                raise PyptoRtError(RuntimeError(
                    f"pypto_amd._host was built against ABI version {_host.ABI_VERSION}, this package needs "
                    f"{ABI_VERSION}: rebuild with `python -m pypto_amd.build`"))
            for op, ptype in _OPS.items():
                if _host.PARAM_BYTES[op] != ctypes.sizeof(ptype):
                    raise PyptoRtError(RuntimeError(f"parameter block of '{op}' differs between Python and pypto_amd._host"))
            addr = lambda f: ctypes.cast(f, ctypes.c_void_p).value
            _host.bind({op: (addr(getattr(_lib, f"pto_{op}_workspace")), addr(getattr(_lib, f"pto_{op}_launch")))
                        for op in _OPS}, addr(_lib.pto_last_error))
            _host_mod = _host
    return _host_mod


_op_ids = {}


def launch(op, tensors, params):
    """Validate, size the workspace, launch on the current stream of the tensors' device: one call into the pybind11
    layer (csrc/host_binding.cpp), which checks the operands the way the reference's binding does
    (python/src/bindings/torch_tensor_converter.cpp:91-214), fills the descriptor list and calls the C ABI."""
    op_id = _op_ids.get(op)
    if op_id is None:
        op_id = _op_ids[op] = load_host().OPS[op]
    try:
        _host_mod.launch(op_id, tensors, bytes(params))
    except _host_mod.BindingError as e:
        raise FeError(RuntimeError(str(e))) from None


def launch_ctypes(op, tensors, params, workspace=None, stream=None, sync=0):
    """The same call through ctypes, every step spelled out: for tests of the C ABI and for callers that bring their own
    workspace or stream (``workspace``: a uint8 tensor of at least the size the workspace query returns)."""
    lib = load_library()
    ws_fn, launch_fn = getattr(lib, f"pto_{op}_workspace"), getattr(lib, f"pto_{op}_launch")
    descs = describe(tensors)
    n = len(tensors)
    dev = tensors[0].device
    pref = ctypes.byref(params)
    ws_bytes = ws_fn(descs, n, pref)
    with torch.cuda.device(dev):
        if workspace is None and ws_bytes:
            workspace = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
        s = torch.cuda.current_stream(dev).cuda_stream if stream is None else stream
        rc = launch_fn(descs, n, pref, workspace.data_ptr() if workspace is not None else None,
                       workspace.numel() if workspace is not None else 0, s, sync)
    if rc != 0:
        raise _STATUS_EXC.get(rc, RuntimeError)(lib.pto_last_error().decode())
    return ws_bytes


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
