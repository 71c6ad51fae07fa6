"""ctypes binding of libdfa3d_hip.so (C ABI declared in include/dfa3d.h).

The library is the product: there is no CPU or pure-PyTorch fallback.  If the
shared object is missing or a tensor is not on a GPU, the call raises.
"""
import contextlib
import ctypes
import os
import threading

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libdfa3d_hip.so")

DFA3D_F32, DFA3D_F64, DFA3D_BF16, DFA3D_BF16G = 0, 1, 2, 3
ABI_VERSION = 9

_P, _I = ctypes.c_void_p, ctypes.c_int
_DIMS7 = [_I] * 7      # B S M (C|D) L Q P
_DIMS8 = [_I] * 8      # B S M C D L Q P


class LaunchOptions(ctypes.Structure):
    """dfa3d_launch_options of include/dfa3d.h: how one call is laid out on the machine (never what it computes)."""
    _fields_ = [("iters", _I), ("vec", _I), ("direct", _I), ("tile", _I), ("block", _I), ("pass_", _I), ("chunk", _I),
                ("clear", _I), ("event_binned", _P)]


_O = ctypes.POINTER(LaunchOptions)

# name -> argument types; every entry point returns int
SIGNATURES = {
    "dfa3d_ms_depth_score_sample_forward": [_P] * 5 + _DIMS7 + [_I, _O, _P],
    "dfa3d_ms_depth_score_sample_backward": [_P] * 8 + [ctypes.c_size_t] + _DIMS7 + [_I, _O, _P],
    "dfa3d_wms_deform_attn_forward": [_P, _P, _I, _P, _P, _I, _P, _P, _P] + _DIMS7 + [_I, _O, _P],
    "dfa3d_wms_deform_attn_backward": [_P, _P, _I, _P, _P, _I, _P, _P, _P, _P, _P, _I, _P, _P, _P, ctypes.c_size_t]
    + _DIMS7 + [_I, _O, _P],
    "dfa3d_fused_forward": [_P] * 10 + _DIMS8 + [_I, _I, _O, _P],
    "dfa3d_pack_dist": [_P, _P, _P, _P, ctypes.c_size_t, _I, _I, _I, _I, _I, _P],
    "dfa3d_fused_backward": [_P] * 14 + [ctypes.c_size_t] + _DIMS8 + [_I, _I, _O, _P],
    "dfa3d_fused_backward_static": [_P] * 13 + _DIMS8 + [_I, _I, _O, _P],
    "dfa3d_rebatch_gather": [_P, ctypes.c_longlong, ctypes.c_longlong, _P, _P, _P, _I, _I, _I, _I, _I, _I, _P],
    "dfa3d_rebatch_combine": [_P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _P],
    "dfa3d_abi_version": [],
}

_lib = None


def lib():
    """Loads the shared library once; raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                f"{LIB_PATH} is missing: build it with `python 3d-deformable-attention_amd/build.py` "
                "(hipcc, --offload-arch=gfx950). There is no fallback implementation.")
        handle = ctypes.CDLL(LIB_PATH)
        for name, argtypes in SIGNATURES.items():
            fn = getattr(handle, name)
            fn.argtypes = argtypes
            fn.restype = ctypes.c_int
        for name, dims in (("dfa3d_fused_backward_workspace_bytes", _DIMS8 + [_I]),
                           ("dfa3d_wms_deform_attn_backward_workspace_bytes", _DIMS7),
                           ("dfa3d_ms_depth_score_sample_backward_workspace_bytes", _DIMS7)):
            fn = getattr(handle, name)
            fn.argtypes = dims + [_I, _O]
            fn.restype = ctypes.c_size_t
        handle.dfa3d_packed_dist_bytes.argtypes = [_I] * 5
        handle.dfa3d_packed_dist_bytes.restype = ctypes.c_size_t
        handle.dfa3d_static_scratch_bytes.argtypes = []
        handle.dfa3d_static_scratch_bytes.restype = ctypes.c_size_t
        handle.dfa3d_last_error.argtypes = []
        handle.dfa3d_last_error.restype = ctypes.c_char_p
        if handle.dfa3d_abi_version() != ABI_VERSION:
            raise ImportError(f"{LIB_PATH}: ABI version {handle.dfa3d_abi_version()} != expected {ABI_VERSION}; rebuild")
        _lib = handle
    return _lib


def check(rc, name):
    if rc != 0:
        msg = lib().dfa3d_last_error().decode("utf-8", "replace")
        raise RuntimeError(f"{name} failed with code {rc}: {msg}")


_tls = threading.local()


@contextlib.contextmanager
def launch_options(**fields):
    """Every library call this thread makes inside the block carries these launch options
    (``iters``, ``vec``, ``direct``, ``tile``, ``block``, ``pass_``, ``chunk``, ``event_binned``); nested blocks
    add to the enclosing ones.  Outside any block calls pass NULL: the defaults."""
    merged = dict(getattr(_tls, "fields", {}))
    for k, v in fields.items():
        if k == "pass":
            k = "pass_"
        if k not in dict(LaunchOptions._fields_):
            raise TypeError(f"unknown launch option {k!r}")
        merged[k] = v
    saved = getattr(_tls, "fields", None)
    _tls.fields = merged
    try:
        yield
    finally:
        if saved is None:
            del _tls.fields
        else:
            _tls.fields = saved


def current_fields():
    """Copy of the calling thread's launch options (what an autograd Function keeps from its forward: the backward
    of a Function with GPU inputs runs on the autograd engine's worker thread, where the caller's ``with
    launch_options(...)`` block is not in force)."""
    return dict(getattr(_tls, "fields", None) or {})


@contextlib.contextmanager
def restored_options(fields):
    """Puts exactly ``fields`` (a dict from ``current_fields``) in force on the calling thread for the block."""
    saved = getattr(_tls, "fields", None)
    _tls.fields = dict(fields)
    try:
        yield
    finally:
        if saved is None:
            del _tls.fields
        else:
            _tls.fields = saved


def options():
    """ctypes argument for the ``opts`` parameter of an entry point: NULL, or the calling thread's current options."""
    fields = getattr(_tls, "fields", None)
    if not fields:
        return None
    return ctypes.pointer(LaunchOptions(**fields))


def dtype_code(t):
    if t.dtype == torch.float32:
        return DFA3D_F32
    if t.dtype == torch.float64:
        return DFA3D_F64
    if t.dtype == torch.bfloat16:
        return DFA3D_BF16
    raise TypeError(f"DFA3D kernels take float32, float64 or bfloat16 storage, got {t.dtype}")


def ptr(t):
    return ctypes.c_void_p(t.data_ptr()) if t is not None else ctypes.c_void_p(0)


def stream_of(t):
    return ctypes.c_void_p(torch.cuda.current_stream(t.device).cuda_stream)
