"""Camera re-batching around the DFA3D operator: the BEV queries that project into each camera are copied into
a per-camera batch before the attention and the per-camera results are averaged back into the BEV slots
afterwards.  The reference does both in python loops over batch x cameras
(BEVFormer_DFA3D/projects/mmdet3d_plugin/bevformer/modules/spatial_cross_attention.py:716-722, 741-748);
here each direction is one HIP kernel (csrc/dfa3d_rebatch.hip), and each kernel is the other's backward."""
import torch
from torch.autograd import Function
from torch.autograd.function import once_differentiable

from . import _lib

__all__ = ["camera_index", "rebatch_gather", "rebatch_combine", "RebatchGatherFunction", "RebatchCombineFunction"]


def camera_index(hit):
    """``hit`` (cams, Nq) bool: query q projects into camera i.  Returns ``index`` (cams, max_len) int32, the
    queries of each camera in ascending order padded with -1, and its inverse ``pos`` (cams, Nq) int32
    (position of q in camera i's list, or -1).  ``max_len`` depends on the data, so this synchronises with the
    device once, like the reference's ``nonzero`` calls (spatial_cross_attention.py:704-707)."""
    cams, Nq = hit.shape
    hit = hit.bool()
    rank = hit.cumsum(1, dtype=torch.int32) - 1                      # position among the camera's queries
    pos = torch.where(hit, rank, torch.full_like(rank, -1)).contiguous()
    max_len = int(hit.sum(1).max().item()) if hit.numel() else 0
    index = torch.full((cams, max(max_len, 1)), -1, dtype=torch.int32, device=hit.device)
    cam, q = hit.nonzero(as_tuple=True)
    index[cam, rank[cam, q].long()] = q.to(torch.int32)
    return index, pos, max_len


def _check(t, name, dtype=None):
    if not t.is_cuda:
        raise RuntimeError(f"{name} must be a CUDA tensor")
    if not t.is_contiguous():
        raise RuntimeError(f"{name} tensor has to be contiguous")
    if dtype is not None and t.dtype != dtype:
        raise RuntimeError(f"{name} has dtype {t.dtype}, expected {dtype}")


def rebatch_gather(src, index, scale=None, per_camera=False):
    """``src`` (bs, Nq, E), or (cams, bs, Nq, E) with ``per_camera`` -> (bs, cams, max_len, E):
    row [j, i, k] = scale[j, q] * src[(i,) j, q] with q = index[i, k], zeros where index is -1."""
    _check(src, "src")
    _check(index, "index", torch.int32)
    cams, max_len = index.shape
    if per_camera:
        if src.dim() != 4 or src.shape[0] != cams:
            raise RuntimeError(f"src must be (cams, bs, Nq, E), got {tuple(src.shape)}")
        _, bs, Nq, E = src.shape
        cam_stride, batch_stride = bs * Nq * E, Nq * E
    else:
        if src.dim() != 3:
            raise RuntimeError(f"src must be (bs, Nq, E), got {tuple(src.shape)}")
        bs, Nq, E = src.shape
        cam_stride, batch_stride = 0, Nq * E
    if scale is not None:
        _check(scale, "scale", src.dtype)
        if tuple(scale.shape) != (bs, Nq):
            raise RuntimeError(f"scale must be (bs, Nq), got {tuple(scale.shape)}")
    dst = torch.empty(bs, cams, max_len, E, dtype=src.dtype, device=src.device)
    if dst.numel() == 0:
        return dst
    with torch.cuda.device(src.device):
        rc = _lib.lib().dfa3d_rebatch_gather(_lib.ptr(src), cam_stride, batch_stride, _lib.ptr(index), _lib.ptr(scale),
                                             _lib.ptr(dst), bs, cams, max_len, Nq, E, _lib.dtype_code(src),
                                             _lib.stream_of(src))
    _lib.check(rc, "dfa3d_rebatch_gather")
    return dst


def rebatch_combine(src, pos, scale=None):
    """``src`` (bs, cams, max_len, E) -> (bs, Nq, E): row [j, q] = scale[j, q] * sum over the cameras i that see q
    of src[j, i, pos[i, q]]."""
    _check(src, "src")
    _check(pos, "pos", torch.int32)
    if src.dim() != 4 or pos.dim() != 2 or src.shape[1] != pos.shape[0]:
        raise RuntimeError(f"src must be (bs, cams, max_len, E) and pos (cams, Nq), got {tuple(src.shape)}, {tuple(pos.shape)}")
    bs, cams, max_len, E = src.shape
    Nq = pos.shape[1]
    if scale is not None:
        _check(scale, "scale", src.dtype)
        if tuple(scale.shape) != (bs, Nq):
            raise RuntimeError(f"scale must be (bs, Nq), got {tuple(scale.shape)}")
    dst = torch.empty(bs, Nq, E, dtype=src.dtype, device=src.device)
    if dst.numel() == 0:
        return dst
    if src.numel() == 0:
        return dst.zero_()
    with torch.cuda.device(src.device):
        rc = _lib.lib().dfa3d_rebatch_combine(_lib.ptr(src), _lib.ptr(pos), _lib.ptr(scale), _lib.ptr(dst), bs, cams,
                                              max_len, Nq, E, _lib.dtype_code(src), _lib.stream_of(src))
    _lib.check(rc, "dfa3d_rebatch_combine")
    return dst


class RebatchGatherFunction(Function):
    """``apply(src (bs, Nq, E), index, pos) -> (bs, cams, max_len, E)``; differentiable in ``src``."""

    @staticmethod
    def forward(ctx, src, index, pos):
        ctx.save_for_backward(pos)
        return rebatch_gather(src.contiguous(), index)

    @staticmethod
    @once_differentiable
    def backward(ctx, grad):
        pos, = ctx.saved_tensors
        return rebatch_combine(grad.contiguous(), pos), None, None


class RebatchCombineFunction(Function):
    """``apply(src (bs, cams, max_len, E), index, pos, scale (bs, Nq) or None) -> (bs, Nq, E)``; differentiable in
    ``src`` (``scale`` is a constant: the reciprocal camera count)."""

    @staticmethod
    def forward(ctx, src, index, pos, scale):
        ctx.save_for_backward(index, scale)
        return rebatch_combine(src.contiguous(), pos, scale)

    @staticmethod
    @once_differentiable
    def backward(ctx, grad):
        index, scale = ctx.saved_tensors
        return rebatch_gather(grad.contiguous(), index, scale), None, None, None
