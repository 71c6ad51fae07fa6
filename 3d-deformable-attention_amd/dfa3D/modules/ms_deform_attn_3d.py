"""The attention module that calls the DFA3D operator in DFA3D-BEVFormer's spatial cross-attention,
without mmcv: same constructor arguments, parameter names (so the reference's checkpoints load with
``load_state_dict``), forward signature and results as ``MSDeformableAttention3D_DFA3D``
(BEVFormer_DFA3D/projects/mmdet3d_plugin/bevformer/modules/spatial_cross_attention.py:409-589, whose
constructor and value / offset / weight layers come from ``MSDeformableAttention3D``, :186-279).

Differences in how the same numbers are produced:
  * the depth distribution goes to the operator as (bs, keys, 1, D); the reference repeats it once per
    head (:496-497);
  * ``weight_update`` (:579) comes out of the operator's kernel; the (bs, Q, heads, L, P, 4) depth-score
    tensor is not materialised unless ``return_depth_score=True`` is passed to ``forward``.
"""
import math
import warnings

import torch
from torch import nn

from ..functional import (MultiScale3DDeformableAttnFunction_fp32,
                          MultiScale3DDeformableAttnWeightUpdateFunction_fp32)

__all__ = ["MSDeformableAttention3D_DFA3D"]


class MSDeformableAttention3D_DFA3D(nn.Module):
    """3D deformable attention over multi-scale image features with per-pixel depth distributions.

    Args (spatial_cross_attention.py:411, :212-221): embed_dims, num_heads, num_levels, num_points (sampling
    points per level and head, over all Z anchors), im2col_step, dropout (unused by the reference's forward as
    well), batch_first, norm_cfg, init_cfg (accepted, unused).
    """

    def __init__(self, embed_dims=256, num_heads=8, num_levels=4, num_points=8, im2col_step=64, dropout=0.1,
                 batch_first=True, norm_cfg=None, init_cfg=None):
        super().__init__()
        if embed_dims % num_heads != 0:
            raise ValueError(f"embed_dims must be divisible by num_heads, but got {embed_dims} and {num_heads}")
        dim_per_head = embed_dims // num_heads
        if dim_per_head & (dim_per_head - 1):
            warnings.warn("a power-of-two dimension per attention head lets every lane of a wavefront carry channels")
        self.norm_cfg = norm_cfg
        self.batch_first = batch_first
        self.output_proj = None
        self.fp16_enabled = False
        self.im2col_step = im2col_step
        self.embed_dims = embed_dims
        self.num_levels = num_levels
        self.num_heads = num_heads
        self.num_points = num_points
        self.sampling_offsets = nn.Linear(embed_dims, num_heads * num_levels * num_points * 2)
        self.attention_weights = nn.Linear(embed_dims, num_heads * num_levels * num_points)
        self.value_proj = nn.Linear(embed_dims, embed_dims)
        self.sampling_offsets_depth = nn.Linear(embed_dims, num_heads * num_levels * num_points)
        self.init_weights()
        self.init_smpl_off_weights()

    def init_weights(self):
        """Zero offset / weight matrices, offset biases on a ring of directions scaled by the point index,
        Xavier-uniform value projection (spatial_cross_attention.py:261-279)."""
        M, L, P = self.num_heads, self.num_levels, self.num_points
        with torch.no_grad():
            self.sampling_offsets.weight.zero_()
            thetas = torch.arange(M, dtype=torch.float32) * (2.0 * math.pi / M)
            ring = torch.stack([thetas.cos(), thetas.sin()], -1)
            ring = ring / ring.abs().max(-1, keepdim=True)[0]
            scale = torch.arange(1, P + 1, dtype=torch.float32).view(1, 1, P, 1)
            self.sampling_offsets.bias.copy_((ring.view(M, 1, 1, 2) * scale).expand(M, L, P, 2).reshape(-1))
            self.attention_weights.weight.zero_()
            self.attention_weights.bias.zero_()
            nn.init.xavier_uniform_(self.value_proj.weight)
            self.value_proj.bias.zero_()

    def init_smpl_off_weights(self):
        """Depth offsets: zero matrix, bias (cos + sin) / 2 of the head's direction times the point index
        (spatial_cross_attention.py:416-427)."""
        M, L, P = self.num_heads, self.num_levels, self.num_points
        with torch.no_grad():
            self.sampling_offsets_depth.weight.zero_()
            thetas = torch.arange(M, dtype=torch.float32) * (2.0 * math.pi / M)
            base = ((thetas.cos() + thetas.sin()) / 2).view(M, 1, 1)
            scale = torch.arange(1, P + 1, dtype=torch.float32).view(1, 1, P)
            self.sampling_offsets_depth.bias.copy_((base * scale).expand(M, L, P).reshape(-1))

    @staticmethod
    def get_spatial_shape_3D(spatial_shape, depth_dim):
        """(L, 2) -> (L, 3) with the number of depth bins as third extent (spatial_cross_attention.py:584-587)."""
        depth = spatial_shape.new_full((*spatial_shape.shape[:-1], 1), depth_dim)
        return torch.cat([spatial_shape, depth], dim=-1).contiguous()

    def pack_dist(self, value_dpt_dist, spatial_shapes, level_start_index):
        """``value_dpt_dist`` (bs, keys, D) laid out for the operator's depth taps (``dfa3D._ext.pack_shared_dist``);
        None where that is not offered.  Valid for as long as the distribution's values do not change."""
        from .. import _ext
        bs, keys, depth = value_dpt_dist.shape
        dist = value_dpt_dist.reshape(bs, keys, 1, depth).to(self.value_proj.weight.dtype).contiguous()
        return _ext.pack_shared_dist(dist, self.get_spatial_shape_3D(spatial_shapes, depth), level_start_index)

    def sampling_locations(self, query, reference_points, spatial_shapes_3D):
        """Normalised (x, y, z) of every sampling point, (bs, Q, heads, L, points, 3): the head's learned
        offsets, divided by the level's (W, H, D), around the query's Z-anchor reference points
        (spatial_cross_attention.py:498-537).  Point p belongs to anchor p % num_Z_anchors."""
        bs, Q, _ = query.shape
        M, L, P = self.num_heads, self.num_levels, self.num_points
        if reference_points.shape[-1] != 3:
            raise ValueError("Last dim of reference_points must be 3 (x, y, depth), but get "
                             f"{reference_points.shape[-1]} instead.")
        Z = reference_points.shape[2]
        if P % Z:
            raise ValueError(f"num_points ({P}) must be a multiple of the number of Z anchors ({Z})")
        uv = self.sampling_offsets(query).view(bs, Q, M, L, P, 2)
        dz = self.sampling_offsets_depth(query).view(bs, Q, M, L, P, 1)
        normalizer = spatial_shapes_3D[:, [1, 0, 2]].to(query.dtype)              # (W, H, D) per level
        offsets = torch.cat([uv, dz], dim=-1) / normalizer[None, None, None, :, None, :]
        anchors = reference_points[:, :, None, None, None, :, :]                   # (bs, Q, 1, 1, 1, Z, 3)
        loc = offsets.view(bs, Q, M, L, P // Z, Z, 3) + anchors
        return loc.view(bs, Q, M, L, P, 3)

    def forward(self, query, key=None, value=None, value_dpt_dist=None, identity=None, query_pos=None,
                key_padding_mask=None, reference_points=None, spatial_shapes=None, level_start_index=None,
                return_depth_score=False, packed_dist=None, **kwargs):
        """Arguments and results as spatial_cross_attention.py:428-583: ``query`` (bs, Q, embed_dims),
        ``value`` (bs, keys, embed_dims), ``value_dpt_dist`` (bs, keys, D), ``reference_points``
        (bs, Q, num_Z_anchors, 3) normalised, ``spatial_shapes`` (L, 2) as (h, w), ``level_start_index`` (L,).
        Returns ``(output (bs, Q, embed_dims), weight_update (bs, Q, heads, 1))``; with
        ``return_depth_score=True`` a third result, the operator's depth scores.  ``packed_dist``: what
        ``self.pack_dist(value_dpt_dist, spatial_shapes, level_start_index)`` returned for this very distribution;
        an encoder that runs several of these layers on one distribution packs once and hands it to each."""
        if value is None:
            value = query
        if query_pos is not None:
            query = query + query_pos
        if not self.batch_first:
            query = query.permute(1, 0, 2)
            value = value.permute(1, 0, 2)
        bs, num_query, _ = query.shape
        num_value = value.shape[1]
        if spatial_shapes.shape[0] != self.num_levels:
            raise ValueError(f"spatial_shapes has {spatial_shapes.shape[0]} levels, the module {self.num_levels}")
        if value_dpt_dist is None or value_dpt_dist.dim() != 3 or value_dpt_dist.shape[:2] != value.shape[:2]:
            raise ValueError("value_dpt_dist must be (bs, num_value, D)")

        value = self.value_proj(value)
        if key_padding_mask is not None:
            value = value.masked_fill(key_padding_mask[..., None], 0.0)
        value = value.view(bs, num_value, self.num_heads, -1)
        dim_depth = value_dpt_dist.shape[2]
        dist = value_dpt_dist.reshape(bs, num_value, 1, dim_depth).to(value.dtype)
        attention_weights = self.attention_weights(query).view(
            bs, num_query, self.num_heads, self.num_levels * self.num_points).softmax(-1)
        attention_weights = attention_weights.view(bs, num_query, self.num_heads, self.num_levels, self.num_points)
        spatial_shapes_3D = self.get_spatial_shape_3D(spatial_shapes, dim_depth)
        sampling_locations = self.sampling_locations(query, reference_points, spatial_shapes_3D)

        if not value.is_cuda:
            raise NotImplementedError("the DFA3D operator runs on the GPU only")
        args = (value.contiguous(), dist.contiguous(), spatial_shapes_3D, level_start_index,
                sampling_locations.contiguous(), attention_weights.contiguous(), self.im2col_step)
        depth_score = None
        if return_depth_score:
            output, depth_score = MultiScale3DDeformableAttnFunction_fp32.apply(*args)
            weight_update = (depth_score.mean(dim=-1) * attention_weights).flatten(-2).sum(dim=-1, keepdim=True)
        else:
            output, weight_update = MultiScale3DDeformableAttnWeightUpdateFunction_fp32.apply(*args, packed_dist)
        if not self.batch_first:
            output = output.permute(1, 0, 2)
        return (output, weight_update, depth_score) if return_depth_score else (output, weight_update)
