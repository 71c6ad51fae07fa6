"""Native entry points of the DFA3D operator, with the names, argument order and keyword
names of the reference's pybind11 module ``dfa3D._ext``
(DFA3D/dfa3D/ops/csrc/pybind.cpp:42-67), backed by the HIP library through its C ABI.

The argument checks are the reference launchers' (contiguity, device, the ``im2col_step``
divisibility rule: DFA3D/dfa3D/ops/csrc/cuda/wms_deform_attn_cuda.cu:220-253,
ms_depth_score_sample_cuda.cu:54-79) plus shape/dtype consistency, which the kernels rely on.
``im2col_step`` has no numeric effect in the reference (it only splits the batch into several
launches); here it is validated and otherwise unused.

Two extra functions, ``dfa3d_fused_forward`` / ``dfa3d_fused_backward``, run both stages in one
kernel each.

Element types: float32 or float64 throughout, or bfloat16 storage (value, distributions,
output, scores in bfloat16; locations, attention weights and every gradient buffer float32).
"""
import contextlib

import torch

from . import _lib

__all__ = [
    "wms_deform_attn_forward", "wms_deform_attn_backward",
    "ms_depth_score_sample_forward", "ms_depth_score_sample_backward",
    "dfa3d_fused_forward", "dfa3d_fused_backward", "fused_backward_grad_dtype", "pack_shared_dist",
]


def _contig(**tensors):
    for name, t in tensors.items():
        if not t.is_contiguous():
            raise RuntimeError(f"{name} tensor has to be contiguous")


def _on_gpu(**tensors):
    dev = None
    for name, t in tensors.items():
        if not t.is_cuda:
            raise RuntimeError(f"{name} must be a CUDA tensor")
        if dev is None:
            dev = t.device
        elif t.device != dev:
            raise RuntimeError(f"{name} is on {t.device}, expected {dev}: all tensors must be on one device")
    return dev


def _step(batch, im2col_step):
    step = min(batch, int(im2col_step))
    if step <= 0 or batch % step != 0:
        raise RuntimeError(f"batch({batch}) must divide im2col_step({step})")
    return step


def _aux_dtype(storage):
    """dtype of locations, attention weights and gradient buffers for a storage dtype."""
    return torch.float32 if storage == torch.bfloat16 else storage


def _expect(t, name, shape=None, dtype=None):
    if shape is not None and tuple(t.shape) != tuple(shape):
        raise RuntimeError(f"{name} has shape {tuple(t.shape)}, expected {tuple(shape)}")
    if dtype is not None and t.dtype != dtype:
        raise RuntimeError(f"{name} has dtype {t.dtype}, expected {dtype}")


def _geometry(shapes, lsi, loc, width, name):
    if shapes.dim() != 2 or shapes.shape[1] != width:
        raise RuntimeError(f"{name}: value_spatial_shapes must be (num_levels, {width}), got {tuple(shapes.shape)}")
    if loc.dim() != 6 or loc.shape[5] != width:
        raise RuntimeError(f"{name}: sampling_locations must be (bs, num_queries, num_heads, num_levels, "
                           f"num_points, {width}), got {tuple(loc.shape)}")
    L = shapes.shape[0]
    _expect(shapes, "value_spatial_shapes", dtype=torch.int64)
    _expect(lsi, "value_level_start_index", shape=(L,), dtype=torch.int64)
    if loc.shape[3] != L:
        raise RuntimeError(f"{name}: sampling_locations has {loc.shape[3]} levels, value_spatial_shapes has {L}")
    return L


def ms_depth_score_sample_forward(value, value_spatial_shapes, value_level_start_index,
                                  sampling_locations, im2col_step):
    """value = depth distributions (bs, num_keys, num_heads, D) -> (bs, Q, heads, L, P, 4)."""
    _contig(value=value, spatial_shapes=value_spatial_shapes, level_start_index=value_level_start_index,
            sampling_loc=sampling_locations)
    dev = _on_gpu(value=value, spatial_shapes=value_spatial_shapes, level_start_index=value_level_start_index,
                  sampling_loc=sampling_locations)
    if value.dim() != 4:
        raise RuntimeError(f"value must be (bs, num_keys, num_heads, D), got {tuple(value.shape)}")
    B, S, M, D = value.shape
    L = _geometry(value_spatial_shapes, value_level_start_index, sampling_locations, 3, "ms_depth_score_sample_forward")
    _, Q, _, _, P, _ = sampling_locations.shape
    _expect(sampling_locations, "sampling_locations", shape=(B, Q, M, L, P, 3), dtype=_aux_dtype(value.dtype))
    _step(B, im2col_step)
    code = _lib.dtype_code(value)
    score = torch.empty(B, Q, M, L, P, 4, dtype=value.dtype, device=dev)
    if score.numel() == 0:
        return score
    with torch.cuda.device(dev):
        rc = _lib.lib().dfa3d_ms_depth_score_sample_forward(
            _lib.ptr(value), _lib.ptr(value_spatial_shapes), _lib.ptr(value_level_start_index),
            _lib.ptr(sampling_locations), _lib.ptr(score), B, S, M, D, L, Q, P, code,
            _lib.options(), _lib.stream_of(value))
    _lib.check(rc, "dfa3d_ms_depth_score_sample_forward")
    return score


def ms_depth_score_sample_backward(value, value_spatial_shapes, value_level_start_index, sampling_locations,
                                   grad_output, grad_value, grad_sampling_loc, im2col_step):
    """Accumulates into ``grad_value`` (pre-zeroed by the caller) and overwrites ``grad_sampling_loc``
    (x and y components are zero: the scores do not depend on x, y inside a pixel cell)."""
    _contig(value=value, spatial_shapes=value_spatial_shapes, level_start_index=value_level_start_index,
            sampling_loc=sampling_locations, grad_output=grad_output, grad_value=grad_value,
            grad_sampling_loc=grad_sampling_loc)
    dev = _on_gpu(value=value, spatial_shapes=value_spatial_shapes, level_start_index=value_level_start_index,
                  sampling_loc=sampling_locations, grad_output=grad_output, grad_value=grad_value,
                  grad_sampling_loc=grad_sampling_loc)
    B, S, M, D = value.shape
    L = _geometry(value_spatial_shapes, value_level_start_index, sampling_locations, 3, "ms_depth_score_sample_backward")
    _, Q, _, _, P, _ = sampling_locations.shape
    aux = _aux_dtype(value.dtype)
    _expect(sampling_locations, "sampling_locations", shape=(B, Q, M, L, P, 3), dtype=aux)
    _expect(grad_output, "grad_output", shape=(B, Q, M, L, P, 4), dtype=value.dtype)
    _expect(grad_value, "grad_value", shape=value.shape, dtype=aux)
    _expect(grad_sampling_loc, "grad_sampling_loc", shape=sampling_locations.shape, dtype=aux)
    _step(B, im2col_step)
    if grad_output.numel() == 0:
        return
    code = _lib.dtype_code(value)
    ws_bytes = _lib.lib().dfa3d_ms_depth_score_sample_backward_workspace_bytes(B, S, M, D, L, Q, P, code, _lib.options())
    workspace = torch.empty(ws_bytes, dtype=torch.uint8, device=dev) if ws_bytes > 0 else None
    with torch.cuda.device(dev):
        rc = _lib.lib().dfa3d_ms_depth_score_sample_backward(
            _lib.ptr(value), _lib.ptr(value_spatial_shapes), _lib.ptr(value_level_start_index),
            _lib.ptr(sampling_locations), _lib.ptr(grad_output), _lib.ptr(grad_value), _lib.ptr(grad_sampling_loc),
            _lib.ptr(workspace), ws_bytes, B, S, M, D, L, Q, P, code, _lib.options(), _lib.stream_of(value))
    _lib.check(rc, "dfa3d_ms_depth_score_sample_backward")


def _wms_dims(value, shapes, lsi, loc, attn, score, name):
    if value.dim() != 4:
        raise RuntimeError(f"value must be (bs, num_keys, num_heads, channels), got {tuple(value.shape)}")
    B, S, M, C = value.shape
    width = shapes.shape[1] if shapes.dim() == 2 else -1
    if width not in (2, 3):
        raise RuntimeError(f"{name}: value_spatial_shapes must be (num_levels, 2) or (num_levels, 3)")
    if loc.dim() != 6 or loc.shape[5] not in (2, 3):
        raise RuntimeError(f"{name}: sampling_locations must end in (num_points, 2|3), got {tuple(loc.shape)}")
    L = shapes.shape[0]
    _expect(shapes, "value_spatial_shapes", dtype=torch.int64)
    _expect(lsi, "value_level_start_index", shape=(L,), dtype=torch.int64)
    _, Q, _, _, P, lw = loc.shape
    aux = _aux_dtype(value.dtype)
    _expect(loc, "sampling_locations", shape=(B, Q, M, L, P, lw), dtype=aux)
    _expect(attn, "attention_weights", shape=(B, Q, M, L, P), dtype=aux)
    if score is not None:
        _expect(score, "depth_scores", shape=(B, Q, M, L, P, 4), dtype=value.dtype)
    return B, S, M, C, L, Q, P, width, lw


def wms_deform_attn_forward(value, value_spatial_shapes, value_level_start_index, sampling_locations,
                            attention_weights, depth_scores, im2col_step):
    """Depth-weighted multi-scale deformable attention -> (bs, num_queries, heads*channels)."""
    _contig(value=value, spatial_shapes=value_spatial_shapes, level_start_index=value_level_start_index,
            sampling_loc=sampling_locations, attn_weight=attention_weights, depth_score=depth_scores)
    dev = _on_gpu(value=value, spatial_shapes=value_spatial_shapes, level_start_index=value_level_start_index,
                  sampling_loc=sampling_locations, attn_weight=attention_weights, depth_score=depth_scores)
    B, S, M, C, L, Q, P, sw, lw = _wms_dims(value, value_spatial_shapes, value_level_start_index, sampling_locations,
                                            attention_weights, depth_scores, "wms_deform_attn_forward")
    _step(B, im2col_step)
    out = torch.empty(B, Q, M * C, dtype=value.dtype, device=dev)
    if out.numel() == 0:
        return out
    with torch.cuda.device(dev):
        rc = _lib.lib().dfa3d_wms_deform_attn_forward(
            _lib.ptr(value), _lib.ptr(value_spatial_shapes), sw, _lib.ptr(value_level_start_index),
            _lib.ptr(sampling_locations), lw, _lib.ptr(attention_weights), _lib.ptr(depth_scores), _lib.ptr(out),
            B, S, M, C, L, Q, P, _lib.dtype_code(value), _lib.options(), _lib.stream_of(value))
    _lib.check(rc, "dfa3d_wms_deform_attn_forward")
    return out


def wms_deform_attn_backward(value, value_spatial_shapes, value_level_start_index, sampling_locations,
                             attention_weights, depth_scores, grad_output, grad_value, grad_sampling_loc,
                             grad_attn_weight, grad_depth_score, im2col_step):
    """Accumulates into ``grad_value`` (pre-zeroed by the caller); overwrites the x, y components of
    ``grad_sampling_loc``, ``grad_attn_weight`` and ``grad_depth_score``.  Names and order of the arguments are the
    reference's (pybind.cpp:48-54)."""
    wms_deform_attn_backward_into(value, value_spatial_shapes, value_level_start_index, sampling_locations,
                                  attention_weights, depth_scores, grad_output, grad_value, grad_sampling_loc,
                                  grad_attn_weight, grad_depth_score, im2col_step, clear=False)


def wms_deform_attn_backward_into(value, value_spatial_shapes, value_level_start_index, sampling_locations,
                                  attention_weights, depth_scores, grad_output, grad_value, grad_sampling_loc,
                                  grad_attn_weight, grad_depth_score, im2col_step, clear=False):
    """``wms_deform_attn_backward`` with one more choice: ``clear=True`` takes a ``grad_value`` that holds anything
    (``torch.empty``) and clears what the kernels add to rather than store (see ``dfa3d_fused_backward``)."""
    _contig(value=value, spatial_shapes=value_spatial_shapes, level_start_index=value_level_start_index,
            sampling_loc=sampling_locations, attn_weight=attention_weights, depth_score=depth_scores,
            grad_output=grad_output, grad_value=grad_value, grad_sampling_loc=grad_sampling_loc,
            grad_attn_weight=grad_attn_weight, grad_depth_score=grad_depth_score)
    dev = _on_gpu(value=value, spatial_shapes=value_spatial_shapes, level_start_index=value_level_start_index,
                  sampling_loc=sampling_locations, attn_weight=attention_weights, depth_score=depth_scores,
                  grad_output=grad_output, grad_value=grad_value, grad_sampling_loc=grad_sampling_loc,
                  grad_attn_weight=grad_attn_weight, grad_depth_score=grad_depth_score)
    B, S, M, C, L, Q, P, sw, lw = _wms_dims(value, value_spatial_shapes, value_level_start_index, sampling_locations,
                                            attention_weights, depth_scores, "wms_deform_attn_backward")
    aux = _aux_dtype(value.dtype)
    if grad_output.numel() != B * Q * M * C:
        raise RuntimeError(f"grad_output has {grad_output.numel()} elements, expected {B * Q * M * C}")
    _expect(grad_output, "grad_output", dtype=value.dtype)
    _expect(grad_value, "grad_value", shape=value.shape, dtype=aux)
    if grad_sampling_loc.dim() != 6 or grad_sampling_loc.shape[5] not in (2, 3):
        raise RuntimeError("grad_sampling_loc must end in (num_points, 2|3)")
    gw = grad_sampling_loc.shape[5]
    _expect(grad_sampling_loc, "grad_sampling_loc", shape=(B, Q, M, L, P, gw), dtype=aux)
    _expect(grad_attn_weight, "grad_attn_weight", shape=(B, Q, M, L, P), dtype=aux)
    _expect(grad_depth_score, "grad_depth_score", shape=(B, Q, M, L, P, 4), dtype=aux)
    _step(B, im2col_step)
    if grad_output.numel() == 0:
        if clear:
            grad_value.zero_()
        return
    code = _lib.dtype_code(value)
    with (_lib.launch_options(clear=1) if clear else contextlib.nullcontext()):
        ws_bytes = _lib.lib().dfa3d_wms_deform_attn_backward_workspace_bytes(B, S, M, C, L, Q, P, code, _lib.options())
        workspace = torch.empty(ws_bytes, dtype=torch.uint8, device=dev) if ws_bytes > 0 else None
        with torch.cuda.device(dev):
            rc = _lib.lib().dfa3d_wms_deform_attn_backward(
                _lib.ptr(value), _lib.ptr(value_spatial_shapes), sw, _lib.ptr(value_level_start_index),
                _lib.ptr(sampling_locations), lw, _lib.ptr(attention_weights), _lib.ptr(depth_scores),
                _lib.ptr(grad_output), _lib.ptr(grad_value), _lib.ptr(grad_sampling_loc), gw,
                _lib.ptr(grad_attn_weight), _lib.ptr(grad_depth_score), _lib.ptr(workspace), ws_bytes, B, S, M, C, L,
                Q, P, code, _lib.options(), _lib.stream_of(value))
    _lib.check(rc, "dfa3d_wms_deform_attn_backward")


def ms_deform_attn_forward(value, value_spatial_shapes, value_level_start_index, sampling_locations,
                           attention_weights, im2col_step):
    """Plain multi-scale deformable attention (every depth score 1): the entry point BEVFormer's temporal
    self-attention and decoder load from mmcv's extension
    (BEVFormer_DFA3D/projects/mmdet3d_plugin/bevformer/modules/multi_scale_deformable_attn_function.py:10-12,:47-53).
    Runs the stage-2 kernel without a score tensor."""
    named = dict(value=value, spatial_shapes=value_spatial_shapes, level_start_index=value_level_start_index,
                 sampling_loc=sampling_locations, attn_weight=attention_weights)
    _contig(**named)
    dev = _on_gpu(**named)
    B, S, M, C, L, Q, P, sw, lw = _wms_dims(value, value_spatial_shapes, value_level_start_index, sampling_locations,
                                            attention_weights, None, "ms_deform_attn_forward")
    _step(B, im2col_step)
    out = torch.empty(B, Q, M * C, dtype=value.dtype, device=dev)
    if out.numel() == 0:
        return out
    with torch.cuda.device(dev):
        rc = _lib.lib().dfa3d_wms_deform_attn_forward(
            _lib.ptr(value), _lib.ptr(value_spatial_shapes), sw, _lib.ptr(value_level_start_index),
            _lib.ptr(sampling_locations), lw, _lib.ptr(attention_weights), None, _lib.ptr(out),
            B, S, M, C, L, Q, P, _lib.dtype_code(value), _lib.options(), _lib.stream_of(value))
    _lib.check(rc, "dfa3d_wms_deform_attn_forward")
    return out


def ms_deform_attn_backward(value, value_spatial_shapes, value_level_start_index, sampling_locations,
                            attention_weights, grad_output, grad_value, grad_sampling_loc, grad_attn_weight,
                            im2col_step, clear=False):
    """Backward of ms_deform_attn_forward (…/multi_scale_deformable_attn_function.py:74-84).  Accumulates into
    ``grad_value`` (pre-zeroed by the caller, or holding anything with ``clear=True``); overwrites
    ``grad_sampling_loc`` and ``grad_attn_weight``."""
    named = dict(value=value, spatial_shapes=value_spatial_shapes, level_start_index=value_level_start_index,
                 sampling_loc=sampling_locations, attn_weight=attention_weights, grad_output=grad_output,
                 grad_value=grad_value, grad_sampling_loc=grad_sampling_loc, grad_attn_weight=grad_attn_weight)
    _contig(**named)
    dev = _on_gpu(**named)
    B, S, M, C, L, Q, P, sw, lw = _wms_dims(value, value_spatial_shapes, value_level_start_index, sampling_locations,
                                            attention_weights, None, "ms_deform_attn_backward")
    aux = _aux_dtype(value.dtype)
    if grad_output.numel() != B * Q * M * C:
        raise RuntimeError(f"grad_output has {grad_output.numel()} elements, expected {B * Q * M * C}")
    _expect(grad_output, "grad_output", dtype=value.dtype)
    _expect(grad_value, "grad_value", shape=value.shape, dtype=aux)
    _expect(grad_sampling_loc, "grad_sampling_loc", shape=sampling_locations.shape, dtype=aux)
    _expect(grad_attn_weight, "grad_attn_weight", shape=(B, Q, M, L, P), dtype=aux)
    _step(B, im2col_step)
    if grad_output.numel() == 0:
        if clear:
            grad_value.zero_()
        return
    code = _lib.dtype_code(value)
    with (_lib.launch_options(clear=1) if clear else contextlib.nullcontext()):
        ws_bytes = _lib.lib().dfa3d_wms_deform_attn_backward_workspace_bytes(B, S, M, C, L, Q, P, code, _lib.options())
        workspace = torch.empty(ws_bytes, dtype=torch.uint8, device=dev) if ws_bytes > 0 else None
        with torch.cuda.device(dev):
            rc = _lib.lib().dfa3d_wms_deform_attn_backward(
                _lib.ptr(value), _lib.ptr(value_spatial_shapes), sw, _lib.ptr(value_level_start_index),
                _lib.ptr(sampling_locations), lw, _lib.ptr(attention_weights), None, _lib.ptr(grad_output),
                _lib.ptr(grad_value), _lib.ptr(grad_sampling_loc), lw, _lib.ptr(grad_attn_weight), None,
                _lib.ptr(workspace), ws_bytes, B, S, M, C, L, Q, P, code, _lib.options(), _lib.stream_of(value))
    _lib.check(rc, "dfa3d_wms_deform_attn_backward")


def _fused_dims(value, dist, shapes3, lsi, loc3, attn, name):
    if value.dim() != 4 or dist.dim() != 4 or value.shape[:2] != dist.shape[:2] or \
            dist.shape[2] not in (1, value.shape[2]):
        raise RuntimeError(f"{name}: value (bs, keys, heads, C) and value_dpt_dist (bs, keys, heads or 1, D) must "
                           f"agree on bs and keys, got {tuple(value.shape)} and {tuple(dist.shape)}")
    _expect(dist, "value_dpt_dist", dtype=value.dtype)
    B, S, M, C = value.shape
    D = dist.shape[3]
    L = _geometry(shapes3, lsi, loc3, 3, name)
    _, Q, _, _, P, _ = loc3.shape
    aux = _aux_dtype(value.dtype)
    _expect(loc3, "sampling_locations", shape=(B, Q, M, L, P, 3), dtype=aux)
    _expect(attn, "attention_weights", shape=(B, Q, M, L, P), dtype=aux)
    return B, S, M, C, D, L, Q, P


def pack_shared_dist(value_dpt_dist, value_spatial_shapes, value_level_start_index):
    """A distribution shared by all heads, (bs, keys, 1, D), laid out for the forward's depth taps (the four pixels
    around every base pixel side by side, per bin): pass the result as ``packed_dist`` to ``dfa3d_fused_forward``.
    Returns None where the library does not offer it (D < 2, float64).  Worth keeping: every forward on the same
    distribution (DFA3D-BEVFormer runs six encoder layers on one) can use the same packed tensor."""
    _contig(value_dpt_dist=value_dpt_dist, spatial_shapes=value_spatial_shapes,
            level_start_index=value_level_start_index)
    dev = _on_gpu(value_dpt_dist=value_dpt_dist, spatial_shapes=value_spatial_shapes,
                  level_start_index=value_level_start_index)
    if value_dpt_dist.dim() != 4 or value_dpt_dist.shape[2] != 1:
        raise RuntimeError(f"value_dpt_dist must be (bs, keys, 1, D), got {tuple(value_dpt_dist.shape)}")
    if value_dpt_dist.dtype == torch.float64:
        return None
    B, S, _, D = value_dpt_dist.shape
    L = value_spatial_shapes.shape[0]
    code = _lib.dtype_code(value_dpt_dist)
    n = _lib.lib().dfa3d_packed_dist_bytes(B, S, D, L, code)
    if n == 0:
        return None
    packed = torch.empty(n, dtype=torch.uint8, device=dev)
    with torch.cuda.device(dev):
        rc = _lib.lib().dfa3d_pack_dist(_lib.ptr(value_dpt_dist), _lib.ptr(value_spatial_shapes),
                                        _lib.ptr(value_level_start_index), _lib.ptr(packed), n, B, S, D, L, code,
                                        _lib.stream_of(value_dpt_dist))
    _lib.check(rc, "dfa3d_pack_dist")
    return packed


def dfa3d_fused_forward(value, value_dpt_dist, value_spatial_shapes, value_level_start_index, sampling_locations,
                        attention_weights, im2col_step, need_depth_score=True, need_weight_update=False,
                        packed_dist=None):
    """One-kernel DFA3D forward -> (output (bs, Q, heads*C), depth_score (bs, Q, heads, L, P, 4) or None), and
    with ``need_weight_update`` a third result, weight_update (bs, Q, heads, 1) = sum over levels and points of
    attention weight * mean corner score.  ``value_dpt_dist`` is (bs, keys, heads, D), or (bs, keys, 1, D) for one
    distribution shared by all heads; for the latter ``packed_dist`` may be what ``pack_shared_dist`` returned for it."""
    _contig(value=value, value_dpt_dist=value_dpt_dist, spatial_shapes=value_spatial_shapes,
            level_start_index=value_level_start_index, sampling_loc=sampling_locations, attn_weight=attention_weights)
    dev = _on_gpu(value=value, value_dpt_dist=value_dpt_dist, spatial_shapes=value_spatial_shapes,
                  level_start_index=value_level_start_index, sampling_loc=sampling_locations,
                  attn_weight=attention_weights)
    B, S, M, C, D, L, Q, P = _fused_dims(value, value_dpt_dist, value_spatial_shapes, value_level_start_index,
                                         sampling_locations, attention_weights, "dfa3d_fused_forward")
    _step(B, im2col_step)
    if packed_dist is not None:
        if value_dpt_dist.shape[2] != 1:
            raise RuntimeError("packed_dist goes with a distribution shared by all heads, (bs, keys, 1, D)")
        need = _lib.lib().dfa3d_packed_dist_bytes(B, S, D, L, _lib.dtype_code(value))
        if need == 0 or packed_dist.device != dev or not packed_dist.is_contiguous() or \
                packed_dist.numel() * packed_dist.element_size() < need:
            raise RuntimeError(f"packed_dist must be a contiguous tensor of at least {need} bytes on {dev}")
    out = torch.empty(B, Q, M * C, dtype=value.dtype, device=dev)
    score = torch.empty(B, Q, M, L, P, 4, dtype=value.dtype, device=dev) if need_depth_score else None
    wu = torch.empty(B, Q, M, 1, dtype=_aux_dtype(value.dtype), device=dev) if need_weight_update else None
    if out.numel() == 0:
        return (out, score, wu) if need_weight_update else (out, score)
    with torch.cuda.device(dev):
        rc = _lib.lib().dfa3d_fused_forward(
            _lib.ptr(value), _lib.ptr(value_dpt_dist), _lib.ptr(value_spatial_shapes),
            _lib.ptr(value_level_start_index), _lib.ptr(sampling_locations), _lib.ptr(attention_weights),
            _lib.ptr(out), _lib.ptr(score), _lib.ptr(wu), _lib.ptr(packed_dist), B, S, M, C, D, L, Q, P,
            value_dpt_dist.shape[2],
            _lib.dtype_code(value), _lib.options(), _lib.stream_of(value))
    _lib.check(rc, "dfa3d_fused_forward")
    return (out, score, wu) if need_weight_update else (out, score)


def fused_backward_grad_dtype(value, value_dpt_dist, sampling_locations):
    """dtype the one-kernel backward can write grad_value / grad_value_dpt_dist in for these operands: bfloat16 for
    bfloat16 storage when the LDS-tile kernels apply (the gradients then need no conversion pass before autograd
    hands them on), else the accumulation type (float32 / float64)."""
    aux = _aux_dtype(value.dtype)
    if value.dtype != torch.bfloat16 or sampling_locations.numel() == 0:
        return aux
    B, S, M, C = value.shape
    _, Q, _, L, P, _ = sampling_locations.shape
    n = _lib.lib().dfa3d_fused_backward_workspace_bytes(B, S, M, C, value_dpt_dist.shape[3], L, Q, P,
                                                        value_dpt_dist.shape[2], _lib.DFA3D_BF16G, _lib.options())
    return torch.bfloat16 if n > 0 else aux


def dfa3d_fused_backward(value, value_dpt_dist, value_spatial_shapes, value_level_start_index, sampling_locations,
                         attention_weights, grad_output, grad_depth_score, grad_value, grad_value_dpt_dist,
                         grad_sampling_loc, grad_attn_weight, im2col_step, grad_weight_update=None, clear=False):
    """One-kernel DFA3D backward.  ``grad_depth_score`` and ``grad_weight_update`` (gradients arriving at the
    depth_score and weight_update outputs) may be None.  Accumulates into ``grad_value`` / ``grad_value_dpt_dist``
    (float32 / float64, or both bfloat16 where ``fused_backward_grad_dtype`` says so): pre-zeroed by the caller as
    the reference's are, or, with ``clear=True``, holding anything (``torch.empty``): the call then clears what its
    kernels add to rather than store, about a quarter of the two buffers on the tile kernels.  Overwrites
    ``grad_sampling_loc`` (…, 3) and ``grad_attn_weight``."""
    named = dict(value=value, value_dpt_dist=value_dpt_dist, spatial_shapes=value_spatial_shapes,
                 level_start_index=value_level_start_index, sampling_loc=sampling_locations,
                 attn_weight=attention_weights, grad_output=grad_output, grad_value=grad_value,
                 grad_value_dpt_dist=grad_value_dpt_dist, grad_sampling_loc=grad_sampling_loc,
                 grad_attn_weight=grad_attn_weight)
    if grad_depth_score is not None:
        named["grad_depth_score"] = grad_depth_score
    if grad_weight_update is not None:
        named["grad_weight_update"] = grad_weight_update
    _contig(**named)
    dev = _on_gpu(**named)
    B, S, M, C, D, L, Q, P = _fused_dims(value, value_dpt_dist, value_spatial_shapes, value_level_start_index,
                                         sampling_locations, attention_weights, "dfa3d_fused_backward")
    aux = _aux_dtype(value.dtype)
    if grad_output.numel() != B * Q * M * C:
        raise RuntimeError(f"grad_output has {grad_output.numel()} elements, expected {B * Q * M * C}")
    _expect(grad_output, "grad_output", dtype=value.dtype)
    if grad_depth_score is not None:
        _expect(grad_depth_score, "grad_depth_score", shape=(B, Q, M, L, P, 4), dtype=value.dtype)
    if grad_weight_update is not None:
        if grad_weight_update.numel() != B * Q * M:
            raise RuntimeError(f"grad_weight_update has {grad_weight_update.numel()} elements, expected {B * Q * M}")
        _expect(grad_weight_update, "grad_weight_update", dtype=aux)
    g16 = value.dtype == torch.bfloat16 and grad_value.dtype == torch.bfloat16
    _expect(grad_value, "grad_value", shape=value.shape, dtype=torch.bfloat16 if g16 else aux)
    _expect(grad_value_dpt_dist, "grad_value_dpt_dist", shape=value_dpt_dist.shape, dtype=torch.bfloat16 if g16 else aux)
    _expect(grad_sampling_loc, "grad_sampling_loc", shape=(B, Q, M, L, P, 3), dtype=aux)
    _expect(grad_attn_weight, "grad_attn_weight", shape=(B, Q, M, L, P), dtype=aux)
    _step(B, im2col_step)
    if grad_output.numel() == 0:
        if clear:
            grad_value.zero_()
            grad_value_dpt_dist.zero_()
        return
    code = _lib.DFA3D_BF16G if g16 else _lib.dtype_code(value)
    with (_lib.launch_options(clear=1) if clear else contextlib.nullcontext()):
        # scratch for the binned (LDS-accumulating) kernels; 0 bytes means the direct kernel is used
        ws_bytes = _lib.lib().dfa3d_fused_backward_workspace_bytes(B, S, M, C, D, L, Q, P, value_dpt_dist.shape[2],
                                                                    code, _lib.options())
        workspace = torch.empty(ws_bytes, dtype=torch.uint8, device=dev) if ws_bytes > 0 else None
        with torch.cuda.device(dev):
            rc = _lib.lib().dfa3d_fused_backward(
                _lib.ptr(value), _lib.ptr(value_dpt_dist), _lib.ptr(value_spatial_shapes),
                _lib.ptr(value_level_start_index), _lib.ptr(sampling_locations), _lib.ptr(attention_weights),
                _lib.ptr(grad_output), _lib.ptr(grad_depth_score), _lib.ptr(grad_weight_update), _lib.ptr(grad_value),
                _lib.ptr(grad_value_dpt_dist), _lib.ptr(grad_sampling_loc), _lib.ptr(grad_attn_weight),
                _lib.ptr(workspace), ws_bytes, B, S, M, C, D, L, Q, P, value_dpt_dist.shape[2], code,
                _lib.options(), _lib.stream_of(value))
    _lib.check(rc, "dfa3d_fused_backward")
