"""DFA3D-BEVFormer's spatial cross-attention without mmcv: ``SpatialCrossAttention_DFA3D``
(BEVFormer_DFA3D/projects/mmdet3d_plugin/bevformer/modules/spatial_cross_attention.py:616-751; constructor and
output projection from ``SpatialCrossAttention``, :54-83).  Same constructor arguments, parameter names
(``output_proj``, ``deformable_attention.*``, ``empty_query``), forward signature and result; the camera
re-batching (python loops over batch x cameras in the reference, :716-722 and :741-748) runs as two HIP kernels
(``dfa3D.rebatch``)."""
import torch
from torch import nn

from ..rebatch import RebatchCombineFunction, RebatchGatherFunction, camera_index, rebatch_gather
from .ms_deform_attn_3d import MSDeformableAttention3D_DFA3D

__all__ = ["SpatialCrossAttention_DFA3D"]


class SpatialCrossAttention_DFA3D(nn.Module):
    """Every camera attends with the BEV queries that project into it; the results are averaged over the cameras
    that see a query, projected, and added to the residual.

    ``deformable_attention`` is a module, or a config dict as in the reference's configs
    (``dict(type='MSDeformableAttention3D_DFA3D', embed_dims=256, num_points=8, num_levels=4)``,
    projects/configs/bevformer/bevformer_base_DFA3D.py) from which the module is built here."""

    def __init__(self, embed_dims=256, num_cams=6, bev_h=200, bev_w=200, use_empty=False, num_head=8, pc_range=None,
                 dropout=0.1, init_cfg=None, batch_first=False, deformable_attention=None, **kwargs):
        super().__init__()
        self.init_cfg = init_cfg
        self.dropout = nn.Dropout(dropout)
        self.pc_range = pc_range
        self.fp16_enabled = False
        if deformable_attention is None:
            deformable_attention = dict(type="MSDeformableAttention3D_DFA3D", embed_dims=embed_dims, num_levels=4)
        if isinstance(deformable_attention, dict):
            cfg = dict(deformable_attention)
            kind = cfg.pop("type", "MSDeformableAttention3D_DFA3D")
            if kind != "MSDeformableAttention3D_DFA3D":
                raise ValueError(f"deformable_attention type {kind!r} is not available here; pass a module instead")
            deformable_attention = MSDeformableAttention3D_DFA3D(**cfg)
        self.deformable_attention = deformable_attention
        self.embed_dims = embed_dims
        self.num_cams = num_cams
        self.output_proj = nn.Linear(embed_dims, embed_dims)
        self.batch_first = batch_first
        self.bev_h = bev_h
        self.bev_w = bev_w
        self.num_head = num_head
        self.use_empty = use_empty
        if use_empty:
            self.empty_query = nn.Embedding(bev_h * bev_w * num_head, embed_dims)
        self.init_weight()

    def init_weight(self):
        """Xavier-uniform output projection, zero bias (spatial_cross_attention.py:80-82)."""
        nn.init.xavier_uniform_(self.output_proj.weight)
        nn.init.zeros_(self.output_proj.bias)

    def forward(self, query, key, value, residual=None, query_pos=None, key_padding_mask=None, reference_points=None,
                spatial_shapes=None, reference_points_cam=None, bev_mask=None, level_start_index=None,
                value_dpt_dist=None, flag="encoder", **kwargs):
        """``query`` (bs, Nq, E); ``key`` / ``value`` (cams, keys, bs, E); ``value_dpt_dist`` (cams, keys, bs, D);
        ``reference_points_cam`` (cams, bs, Nq, Z, 3) normalised image coordinates and depth of the Z anchors of
        every BEV query in every camera; ``bev_mask`` (cams, bs, Nq, Z) which of them fall inside the image.
        Returns (bs, Nq, E).  As in the reference, the queries of a camera are those whose mask is set for the
        first batch element (:704-706), while the averaging counts cameras per batch element (:745-748)."""
        if key is None:
            key = query
        if value is None:
            value = key
        inp_residual = query if residual is None else residual
        if query_pos is not None:
            query = query + query_pos
        bs, num_query, _ = query.shape
        Z = reference_points_cam.size(3)
        cams = self.num_cams

        hit = bev_mask[:, 0].sum(-1) > 0                                         # (cams, Nq)
        index, pos, max_len = camera_index(hit)
        queries_rebatch = RebatchGatherFunction.apply(query, index, pos)         # (bs, cams, max_len, E)
        ref = reference_points_cam.to(query.dtype).reshape(cams, bs, num_query, Z * 3).contiguous()
        reference_points_rebatch = rebatch_gather(ref, index, per_camera=True)   # (bs, cams, max_len, Z*3)
        L = index.shape[1]

        keys = key.shape[1]
        key = key.permute(2, 0, 1, 3).reshape(bs * cams, keys, self.embed_dims)
        value = value.permute(2, 0, 1, 3).reshape(bs * cams, keys, self.embed_dims)
        value_dpt_dist = value_dpt_dist.permute(2, 0, 1, 3).reshape(bs * cams, keys, value_dpt_dist.shape[-1])

        queries, update_weight = self.deformable_attention(
            query=queries_rebatch.view(bs * cams, L, self.embed_dims), key=key, value=value,
            value_dpt_dist=value_dpt_dist, reference_points=reference_points_rebatch.view(bs * cams, L, Z, 3),
            spatial_shapes=spatial_shapes, level_start_index=level_start_index, **kwargs)
        queries = queries.reshape(bs, cams, L, self.embed_dims)
        if self.use_empty:
            # learned per-(BEV cell, head) embedding for what the depth-weighted sampling left unexplained (:739-740)
            update_weight = update_weight.view(bs, cams, L, *update_weight.shape[2:])
            table = self.empty_query.weight.view(self.bev_h * self.bev_w, self.num_head, self.embed_dims)
            valid = (index >= 0)
            empty = table[index.clamp(min=0).long()] * valid[..., None, None].to(table.dtype)   # (cams, L, heads, E)
            queries = queries + ((1 - update_weight) * empty[None]).mean(dim=-2)

        count = (bev_mask.sum(-1) > 0).permute(1, 2, 0).sum(-1)                  # (bs, Nq) cameras seeing each query
        scale = (1.0 / torch.clamp(count, min=1.0)).to(queries.dtype).contiguous()
        slots = RebatchCombineFunction.apply(queries, index, pos, scale)         # (bs, Nq, E)
        slots = self.output_proj(slots)
        return self.dropout(slots) + inp_residual
