"""TEST INFRASTRUCTURE ONLY: ctypes front end of the CPU restatement in
``dfa3d_oracle.c`` (built by ``oracle/Makefile`` into ``libdfa3d_oracle.so``).

Only the test-suite, the smoke check and the benchmark's CPU-baseline leg may
import this module; the shipped package never does.

The four kernels mirror the reference's four native entry points
(DFA3D/dfa3D/ops/csrc/pybind.cpp:42-67); ``dfa3d_forward`` / ``dfa3d_backward``
compose them the way the reference's one-stage autograd Function does
(BEVFormer_DFA3D/projects/mmdet3d_plugin/bevformer/modules/
multi_scale_3ddeformable_attn_function.py:279-303 and :306-352).

All arguments are contiguous CPU ``torch`` tensors, float32 or float64
(shapes/level starts int64), the two types the reference dispatches.
"""
import contextlib
import ctypes
import os
import subprocess

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libdfa3d_oracle.so")
_lib = None


def build(force=False):
    """Compile the C restatement with gcc (seconds)."""
    args = ["make", "-C", _HERE]
    if force:
        args.insert(1, "-B")
    subprocess.run(args, check=True, stdout=subprocess.DEVNULL)


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = ctypes.CDLL(_LIB_PATH)
        _lib.dfa3d_oracle_set_threads.restype = ctypes.c_int
        _lib.dfa3d_oracle_get_threads.restype = ctypes.c_int
    return _lib


def set_threads(n):
    return lib().dfa3d_oracle_set_threads(ctypes.c_int(int(n)))


def get_threads():
    return lib().dfa3d_oracle_get_threads()


_float_geometry = False


@contextlib.contextmanager
def float_geometry():
    """Inside the block, float64 calls use the float32 path's pixel coordinates (the locations must be float32
    values held in float64): their sums are then the exact sums of the terms the float32 path adds up."""
    global _float_geometry
    saved, _float_geometry = _float_geometry, True
    try:
        yield
    finally:
        _float_geometry = saved


def _suffix(t):
    if t.dtype == torch.float32:
        return "f32"
    if t.dtype == torch.float64:
        return "f64g32" if _float_geometry else "f64"
    raise TypeError(f"oracle handles float32/float64 only, got {t.dtype}")


def _p(t):
    assert t.device.type == "cpu" and t.is_contiguous(), "oracle needs contiguous CPU tensors"
    return ctypes.c_void_p(t.data_ptr())


def _i(*xs):
    return [ctypes.c_int(int(x)) for x in xs]


def _check_same(*ts):
    for t in ts[1:]:
        assert t.dtype == ts[0].dtype, "oracle operands must share one floating type"


def depth_score_forward(dist, shapes3, lsi, loc3):
    """(B,S,M,D), (L,3), (L,), (B,Q,M,L,P,3) -> score (B,Q,M,L,P,4)."""
    _check_same(dist, loc3)
    B, S, M, D = dist.shape
    _, Q, _, L, P, three = loc3.shape
    assert three == 3 and shapes3.shape == (L, 3) and shapes3.dtype == torch.int64
    score = torch.empty(B, Q, M, L, P, 4, dtype=dist.dtype)
    fn = getattr(lib(), "dfa3d_oracle_depth_score_forward_" + _suffix(dist))
    fn(_p(dist), _p(shapes3), _p(lsi), _p(loc3), *_i(B, S, M, D, L, Q, P), _p(score))
    return score


def depth_score_backward(dist, shapes3, lsi, loc3, grad_score):
    """-> (grad_dist, grad_loc3); grad_loc3[..., :2] is identically zero."""
    _check_same(dist, loc3, grad_score)
    B, S, M, D = dist.shape
    _, Q, _, L, P, _ = loc3.shape
    grad_dist = torch.zeros_like(dist)
    grad_loc = torch.empty_like(loc3)
    fn = getattr(lib(), "dfa3d_oracle_depth_score_backward_" + _suffix(dist))
    fn(_p(dist), _p(shapes3), _p(lsi), _p(loc3), _p(grad_score.contiguous()),
       *_i(B, S, M, D, L, Q, P), _p(grad_dist), _p(grad_loc))
    return grad_dist, grad_loc


def wms_forward(value, shapes, lsi, loc, attn, score):
    """value (B,S,M,C); shapes (L,2|3); loc (B,Q,M,L,P,2|3) -> out (B,Q,M*C)."""
    _check_same(value, loc, attn, score)
    B, S, M, C = value.shape
    _, Q, _, L, P, ls = loc.shape
    out = torch.empty(B, Q, M * C, dtype=value.dtype)
    fn = getattr(lib(), "dfa3d_oracle_wms_forward_" + _suffix(value))
    fn(_p(value), _p(shapes), ctypes.c_int(shapes.shape[1]), _p(lsi), _p(loc), ctypes.c_int(ls),
       _p(attn), _p(score), *_i(B, S, M, C, L, Q, P), _p(out))
    return out


def wms_backward(value, shapes, lsi, loc, attn, score, grad_out):
    """-> (grad_value, grad_loc_xy (B,Q,M,L,P,2), grad_attn, grad_score)."""
    _check_same(value, loc, attn, score, grad_out)
    B, S, M, C = value.shape
    _, Q, _, L, P, ls = loc.shape
    grad_value = torch.zeros_like(value)
    grad_loc = torch.empty(B, Q, M, L, P, 2, dtype=value.dtype)
    grad_attn = torch.empty_like(attn)
    grad_score = torch.empty_like(score)
    fn = getattr(lib(), "dfa3d_oracle_wms_backward_" + _suffix(value))
    fn(_p(value), _p(shapes), ctypes.c_int(shapes.shape[1]), _p(lsi), _p(loc), ctypes.c_int(ls),
       _p(attn), _p(score), _p(grad_out.contiguous()), *_i(B, S, M, C, L, Q, P),
       _p(grad_value), _p(grad_loc), ctypes.c_int(2), _p(grad_attn), _p(grad_score))
    return grad_value, grad_loc, grad_attn, grad_score


def dfa3d_forward(value, dist, shapes3, lsi, loc3, attn):
    """One-stage DFA3D forward -> (output (B,Q,M*C), depth_score)."""
    score = depth_score_forward(dist, shapes3, lsi, loc3)
    out = wms_forward(value, shapes3, lsi, loc3, attn, score)
    return out, score


def dfa3d_backward(value, dist, shapes3, lsi, loc3, attn, score, grad_out):
    """One-stage DFA3D backward -> (grad_value, grad_dist, grad_loc3, grad_attn)."""
    grad_value, grad_xy, grad_attn, grad_score = wms_backward(
        value, shapes3, lsi, loc3, attn, score, grad_out)
    grad_dist, grad_loc = depth_score_backward(dist, shapes3, lsi, loc3, grad_score)
    grad_loc[..., :2] = grad_loc[..., :2] + grad_xy
    return grad_value, grad_dist, grad_loc, grad_attn
