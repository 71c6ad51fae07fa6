"""DFA3D (3D deformable attention) operator for AMD MI355X.

Import layout of the reference's standalone package is kept so that its callers work unchanged:
``from dfa3D.ops.multi_scale_3D_deform_attn import ...`` (unittest_DFA3D.py:3-6) and
``from dfa3D import ext_loader; ext_loader.load_ext('_ext', [...])``
(BEVFormer_DFA3D/projects/mmdet3d_plugin/bevformer/modules/multi_scale_3ddeformable_attn_function.py:20-22).
"""
from . import ext_loader  # noqa: F401
from .functional import *  # noqa: F401,F403
from .functional import __all__ as _functions

__all__ = ["ext_loader"] + list(_functions)
__version__ = "0.1.0"
