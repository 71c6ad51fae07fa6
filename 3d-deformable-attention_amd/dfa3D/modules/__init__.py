from .ms_deform_attn_3d import MSDeformableAttention3D_DFA3D
from .spatial_cross_attention import SpatialCrossAttention_DFA3D

__all__ = ["MSDeformableAttention3D_DFA3D", "SpatialCrossAttention_DFA3D"]
