"""Autograd surface of the DFA3D operator on MI355X.

Same class names, positional signatures, output shapes and ``None`` pattern of the gradients as
the reference's three Functions
(DFA3D/dfa3D/ops/multi_scale_3D_deform_attn.py:22-221 and, for the one-stage Function, the
corrected version BEVFormer calls:
BEVFormer_DFA3D/projects/mmdet3d_plugin/bevformer/modules/multi_scale_3ddeformable_attn_function.py:276-352):

* ``MultiScaleDepthScoreSampleFunction.apply(value_dpt_dist, spatial_shapes_3D, level_start_index,
  sampling_locations[x,y,z], im2col_step) -> depth_score``
* ``WeightedMultiScaleDeformableAttnFunction.apply(value, spatial_shapes, level_start_index,
  sampling_locations[x,y], attention_weights, depth_score, im2col_step) -> output``
* ``MultiScale3DDeformableAttnFunction.apply(value, value_dpt_dist, spatial_shapes_3D, level_start_index,
  sampling_locations[x,y,z], attention_weights, im2col_step) -> (output, depth_score)``

and their ``_fp32`` / ``_fp16`` twins.  Differences from the reference, all on purpose:

* the one-stage Function runs ONE kernel forward and ONE backward (the reference: two kernels and two
  slice copies forward; two kernels, six zero fills and a device-to-host synchronisation backward);
* a gradient arriving at the ``depth_score`` output is chained into the distribution and z gradients
  (the reference raises ``NotImplementedError`` when it is non-zero, after a host synchronisation);
* the one-stage backward follows the plugin version; the standalone package's own one-stage
  backward (multi_scale_3D_deform_attn.py:167-221) returns a wrong number of gradients and drops the
  x, y terms;
* the ``_fp16`` twins cast to float32 under autocast: the reference's kernels are only instantiated
  for float and double (wms_deform_attn_cuda.cu:267), so its float16 twins cannot run at all;
* bfloat16 ``value`` / ``value_dpt_dist`` (with float32 locations and attention weights) are accepted:
  outputs come back in bfloat16; gradients are accumulated in float32 and, in the one-kernel backward, rounded to
  bfloat16 as the tiles are written (elsewhere: float32 buffers, cast on return).
"""
import functools

import torch
from torch.autograd.function import Function, once_differentiable

from . import _ext, _lib

__all__ = [
    "MultiScaleDepthScoreSampleFunction", "WeightedMultiScaleDeformableAttnFunction",
    "MultiScale3DDeformableAttnFunction",
    "MultiScaleDepthScoreSampleFunction_fp32", "WeightedMultiScaleDeformableAttnFunction_fp32",
    "MultiScale3DDeformableAttnFunction_fp32",
    "MultiScaleDepthScoreSampleFunction_fp16", "WeightedMultiScaleDeformableAttnFunction_fp16",
    "MultiScale3DDeformableAttnFunction_fp16",
    "MultiScale3DDeformableAttnWeightUpdateFunction", "MultiScale3DDeformableAttnWeightUpdateFunction_fp32",
    "MultiScaleDeformableAttnFunction", "MultiScaleDeformableAttnFunction_fp32", "MultiScaleDeformableAttnFunction_fp16",
]


def _aux(t):
    return torch.float32 if t.dtype == torch.bfloat16 else t.dtype


def _packed_for_forward(value_dpt_dist, value_spatial_shapes, value_level_start_index, sampling_locations):
    """The packed form of a distribution shared by all heads when making it pays for this call (its cost grows
    with keys x bins, what it saves with the number of sampling points), else None."""
    if value_dpt_dist.dim() != 4 or value_dpt_dist.shape[2] != 1 or not value_dpt_dist.is_cuda:
        return None
    B, S, _, D = value_dpt_dist.shape
    if sampling_locations.numel() // 3 < B * S * D:
        return None
    return _ext.pack_shared_dist(value_dpt_dist, value_spatial_shapes, value_level_start_index)


def _with_forward_options(backward):
    """Runs a Function's backward under the launch options that were in force when its forward ran.  PyTorch calls
    the backward of a Function with GPU inputs from the autograd engine's per-device thread, and launch options are
    per thread: without this a ``with dfa3D._lib.launch_options(...)`` block around forward and ``.backward()``
    would reach the forward kernels only."""
    @functools.wraps(backward)
    def wrapped(ctx, *grads):
        with _lib.restored_options(getattr(ctx, "launch_fields", {})):
            return backward(ctx, *grads)
    return wrapped


def _grad_in(g, like):
    """Incoming gradient as a contiguous tensor of the dtype the forward output had."""
    g = g.contiguous()
    return g if g.dtype == like else g.to(like)


class MultiScaleDepthScoreSampleFunction(Function):
    """Stage 1: depth scores of the four pixels around every sampling point."""

    @staticmethod
    def forward(ctx, value, value_spatial_shapes, value_level_start_index, sampling_locations, im2col_step):
        ctx.im2col_step = im2col_step
        ctx.launch_fields = _lib.current_fields()      # the backward runs on another thread: see _with_forward_options
        output = _ext.ms_depth_score_sample_forward(
            value, value_spatial_shapes, value_level_start_index, sampling_locations,
            im2col_step=ctx.im2col_step)
        ctx.save_for_backward(value, value_spatial_shapes, value_level_start_index, sampling_locations)
        return output

    @staticmethod
    @once_differentiable
    @_with_forward_options
    def backward(ctx, grad_output):
        value, value_spatial_shapes, value_level_start_index, sampling_locations = ctx.saved_tensors
        grad_value = torch.zeros(value.shape, dtype=_aux(value), device=value.device)
        grad_sampling_loc = torch.empty_like(sampling_locations)
        _ext.ms_depth_score_sample_backward(
            value, value_spatial_shapes, value_level_start_index, sampling_locations,
            _grad_in(grad_output, value.dtype), grad_value, grad_sampling_loc, im2col_step=ctx.im2col_step)
        return grad_value.to(value.dtype), None, None, grad_sampling_loc, None


class WeightedMultiScaleDeformableAttnFunction(Function):
    """Stage 2: multi-scale deformable attention with every corner weighted by its depth score."""

    @staticmethod
    def forward(ctx, value, value_spatial_shapes, value_level_start_index, sampling_locations,
                attention_weights, depth_score, im2col_step):
        ctx.im2col_step = im2col_step
        ctx.launch_fields = _lib.current_fields()      # the backward runs on another thread: see _with_forward_options
        output = _ext.wms_deform_attn_forward(
            value, value_spatial_shapes, value_level_start_index, sampling_locations, attention_weights,
            depth_score, im2col_step=ctx.im2col_step)
        ctx.save_for_backward(value, value_spatial_shapes, value_level_start_index, sampling_locations,
                              attention_weights, depth_score)
        return output

    @staticmethod
    @once_differentiable
    @_with_forward_options
    def backward(ctx, grad_output):
        value, value_spatial_shapes, value_level_start_index, sampling_locations, attention_weights, \
            depth_score = ctx.saved_tensors
        aux = _aux(value)
        grad_value = torch.empty(value.shape, dtype=aux, device=value.device)      # cleared by the call (clear=True)
        grad_sampling_loc = torch.empty_like(sampling_locations)
        if sampling_locations.shape[-1] > 2:
            grad_sampling_loc[..., 2:] = 0
        grad_attn_weight = torch.empty_like(attention_weights)
        grad_depth_score = torch.empty(depth_score.shape, dtype=aux, device=value.device)
        _ext.wms_deform_attn_backward_into(
            value, value_spatial_shapes, value_level_start_index, sampling_locations, attention_weights,
            depth_score, _grad_in(grad_output, value.dtype), grad_value, grad_sampling_loc, grad_attn_weight,
            grad_depth_score, im2col_step=ctx.im2col_step, clear=True)
        return grad_value.to(value.dtype), None, None, grad_sampling_loc, grad_attn_weight, \
            grad_depth_score.to(depth_score.dtype), None


class MultiScaleDeformableAttnFunction(Function):
    """Plain (2-D) multi-scale deformable attention: stage 2 with every depth score equal to 1.  Same signature
    as the Function BEVFormer's temporal self-attention and decoder cross-attention use
    (BEVFormer_DFA3D/projects/mmdet3d_plugin/bevformer/modules/multi_scale_deformable_attn_function.py:90-163)."""

    @staticmethod
    def forward(ctx, value, value_spatial_shapes, value_level_start_index, sampling_locations,
                attention_weights, im2col_step):
        ctx.im2col_step = im2col_step
        ctx.launch_fields = _lib.current_fields()      # the backward runs on another thread: see _with_forward_options
        output = _ext.ms_deform_attn_forward(value, value_spatial_shapes, value_level_start_index,
                                             sampling_locations, attention_weights, im2col_step=ctx.im2col_step)
        ctx.save_for_backward(value, value_spatial_shapes, value_level_start_index, sampling_locations,
                              attention_weights)
        return output

    @staticmethod
    @once_differentiable
    @_with_forward_options
    def backward(ctx, grad_output):
        value, value_spatial_shapes, value_level_start_index, sampling_locations, attention_weights = \
            ctx.saved_tensors
        grad_value = torch.empty(value.shape, dtype=_aux(value), device=value.device)   # cleared by the call
        grad_sampling_loc = torch.empty_like(sampling_locations)
        if sampling_locations.shape[-1] > 2:
            grad_sampling_loc[..., 2:] = 0
        grad_attn_weight = torch.empty_like(attention_weights)
        _ext.ms_deform_attn_backward(
            value, value_spatial_shapes, value_level_start_index, sampling_locations, attention_weights,
            _grad_in(grad_output, value.dtype), grad_value, grad_sampling_loc, grad_attn_weight,
            im2col_step=ctx.im2col_step, clear=True)
        return grad_value.to(value.dtype), None, None, grad_sampling_loc, grad_attn_weight, None


class MultiScale3DDeformableAttnFunction(Function):
    """One-stage DFA3D: returns ``(output, depth_score)``."""

    @staticmethod
    def forward(ctx, value, value_dpt_dist, value_spatial_shapes, value_level_start_index,
                sampling_locations, attention_weights, im2col_step):
        ctx.im2col_step = im2col_step
        ctx.launch_fields = _lib.current_fields()      # the backward runs on another thread: see _with_forward_options
        ctx.set_materialize_grads(False)
        output, depth_score = _ext.dfa3d_fused_forward(
            value, value_dpt_dist, value_spatial_shapes, value_level_start_index, sampling_locations,
            attention_weights, im2col_step=ctx.im2col_step,
            packed_dist=_packed_for_forward(value_dpt_dist, value_spatial_shapes, value_level_start_index,
                                            sampling_locations))
        ctx.save_for_backward(value, value_dpt_dist, value_spatial_shapes, value_level_start_index,
                              sampling_locations, attention_weights)
        return output, depth_score

    @staticmethod
    @once_differentiable
    @_with_forward_options
    def backward(ctx, grad_output, grad_depth_score):
        value, value_dpt_dist, value_spatial_shapes, value_level_start_index, sampling_locations, \
            attention_weights = ctx.saved_tensors
        if grad_output is None:
            grad_output = torch.zeros(value.shape[0], sampling_locations.shape[1], value.shape[2] * value.shape[3],
                                      dtype=value.dtype, device=value.device)
        gdt = _ext.fused_backward_grad_dtype(value, value_dpt_dist, sampling_locations)
        # not zeroed here: the call clears the part of the two buffers that its kernels add to (clear=True)
        grad_value = torch.empty(value.shape, dtype=gdt, device=value.device)
        grad_value_dpt_dist = torch.empty(value_dpt_dist.shape, dtype=gdt, device=value.device)
        grad_sampling_loc = torch.empty_like(sampling_locations)
        grad_attn_weight = torch.empty_like(attention_weights)
        _ext.dfa3d_fused_backward(
            value, value_dpt_dist, value_spatial_shapes, value_level_start_index, sampling_locations,
            attention_weights, _grad_in(grad_output, value.dtype),
            None if grad_depth_score is None else _grad_in(grad_depth_score, value.dtype),
            grad_value, grad_value_dpt_dist, grad_sampling_loc, grad_attn_weight, im2col_step=ctx.im2col_step,
            clear=True)
        return grad_value.to(value.dtype), grad_value_dpt_dist.to(value_dpt_dist.dtype), None, None, \
            grad_sampling_loc, grad_attn_weight, None


class MultiScale3DDeformableAttnWeightUpdateFunction(Function):
    """One-stage DFA3D that returns ``(output, weight_update)`` instead of the depth scores:
    ``weight_update`` (bs, Q, heads, 1) is the reduction the reference's caller applies to the score tensor,
    ``(depth_score.mean(-1) * attention_weights).flatten(-2).sum(-1, keepdim=True)``
    (BEVFormer_DFA3D/projects/mmdet3d_plugin/bevformer/modules/spatial_cross_attention.py:579), computed in the
    kernel so that the (bs, Q, heads, L, P, 4) score tensor is never written.  ``value_dpt_dist`` may be
    (bs, keys, 1, D): one distribution for all heads, without the repeat of spatial_cross_attention.py:496-497.
    Both outputs are differentiable.  An optional eighth argument is that distribution as
    ``dfa3D._ext.pack_shared_dist`` lays it out for the forward's depth taps: a caller that runs several layers on
    one distribution (DFA3D-BEVFormer's six encoder layers) packs once and passes it to each; without it the
    forward packs for itself when that pays."""

    @staticmethod
    def forward(ctx, value, value_dpt_dist, value_spatial_shapes, value_level_start_index,
                sampling_locations, attention_weights, im2col_step, packed_dist=None):
        ctx.im2col_step = im2col_step
        ctx.launch_fields = _lib.current_fields()      # the backward runs on another thread: see _with_forward_options
        ctx.set_materialize_grads(False)
        if packed_dist is None:
            packed_dist = _packed_for_forward(value_dpt_dist, value_spatial_shapes, value_level_start_index,
                                              sampling_locations)
        output, _, weight_update = _ext.dfa3d_fused_forward(
            value, value_dpt_dist, value_spatial_shapes, value_level_start_index, sampling_locations,
            attention_weights, im2col_step=ctx.im2col_step, need_depth_score=False, need_weight_update=True,
            packed_dist=packed_dist)
        ctx.save_for_backward(value, value_dpt_dist, value_spatial_shapes, value_level_start_index,
                              sampling_locations, attention_weights)
        return output, weight_update.to(attention_weights.dtype)

    @staticmethod
    @once_differentiable
    @_with_forward_options
    def backward(ctx, grad_output, grad_weight_update):
        value, value_dpt_dist, value_spatial_shapes, value_level_start_index, sampling_locations, \
            attention_weights = ctx.saved_tensors
        aux = _aux(value)
        if grad_output is None:
            grad_output = torch.zeros(value.shape[0], sampling_locations.shape[1], value.shape[2] * value.shape[3],
                                      dtype=value.dtype, device=value.device)
        gdt = _ext.fused_backward_grad_dtype(value, value_dpt_dist, sampling_locations)
        grad_value = torch.empty(value.shape, dtype=gdt, device=value.device)
        grad_value_dpt_dist = torch.empty(value_dpt_dist.shape, dtype=gdt, device=value.device)
        grad_sampling_loc = torch.empty_like(sampling_locations)
        grad_attn_weight = torch.empty_like(attention_weights)
        _ext.dfa3d_fused_backward(
            value, value_dpt_dist, value_spatial_shapes, value_level_start_index, sampling_locations,
            attention_weights, _grad_in(grad_output, value.dtype), None,
            grad_value, grad_value_dpt_dist, grad_sampling_loc, grad_attn_weight, im2col_step=ctx.im2col_step,
            grad_weight_update=None if grad_weight_update is None else _grad_in(grad_weight_update, aux),
            clear=True)
        # one gradient per forward argument: seven, or eight when the packed distribution was passed in
        return (grad_value.to(value.dtype), grad_value_dpt_dist.to(value_dpt_dist.dtype), None, None,
                grad_sampling_loc, grad_attn_weight, None, None)


def _autocast_twin(base, name, doc):
    """Subclass whose forward casts floating inputs to float32 under ``torch.autocast`` (what the
    reference's ``custom_fwd(cast_inputs=torch.float32)`` twins do) and runs outside autocast."""

    def forward(ctx, *args):
        if torch.is_autocast_enabled():
            args = tuple(a.float() if torch.is_tensor(a) and a.is_floating_point() else a for a in args)
            with torch.autocast(device_type="cuda", enabled=False):
                return base.forward(ctx, *args)
        return base.forward(ctx, *args)

    def backward(ctx, *grads):
        with torch.autocast(device_type="cuda", enabled=False):
            return base.backward(ctx, *grads)

    return type(name, (base,), {"forward": staticmethod(forward), "backward": staticmethod(backward),
                                "__doc__": doc, "__module__": __name__})


_FP32_DOC = "Autocast-safe twin: inputs are cast to float32 when autocast is on."
_FP16_DOC = ("Kept for import compatibility. The reference's float16 twin cannot run (its kernels exist for float and "
             "double only); this one behaves like the float32 twin.")

MultiScaleDepthScoreSampleFunction_fp32 = _autocast_twin(
    MultiScaleDepthScoreSampleFunction, "MultiScaleDepthScoreSampleFunction_fp32", _FP32_DOC)
WeightedMultiScaleDeformableAttnFunction_fp32 = _autocast_twin(
    WeightedMultiScaleDeformableAttnFunction, "WeightedMultiScaleDeformableAttnFunction_fp32", _FP32_DOC)
MultiScale3DDeformableAttnFunction_fp32 = _autocast_twin(
    MultiScale3DDeformableAttnFunction, "MultiScale3DDeformableAttnFunction_fp32", _FP32_DOC)
MultiScaleDepthScoreSampleFunction_fp16 = _autocast_twin(
    MultiScaleDepthScoreSampleFunction, "MultiScaleDepthScoreSampleFunction_fp16", _FP16_DOC)
WeightedMultiScaleDeformableAttnFunction_fp16 = _autocast_twin(
    WeightedMultiScaleDeformableAttnFunction, "WeightedMultiScaleDeformableAttnFunction_fp16", _FP16_DOC)
MultiScale3DDeformableAttnFunction_fp16 = _autocast_twin(
    MultiScale3DDeformableAttnFunction, "MultiScale3DDeformableAttnFunction_fp16", _FP16_DOC)
MultiScale3DDeformableAttnWeightUpdateFunction_fp32 = _autocast_twin(
    MultiScale3DDeformableAttnWeightUpdateFunction, "MultiScale3DDeformableAttnWeightUpdateFunction_fp32", _FP32_DOC)
MultiScaleDeformableAttnFunction_fp32 = _autocast_twin(
    MultiScaleDeformableAttnFunction, "MultiScaleDeformableAttnFunction_fp32", _FP32_DOC)
MultiScaleDeformableAttnFunction_fp16 = _autocast_twin(
    MultiScaleDeformableAttnFunction, "MultiScaleDeformableAttnFunction_fp16", _FP16_DOC)
