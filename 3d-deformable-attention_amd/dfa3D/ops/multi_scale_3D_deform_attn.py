"""Import path of the reference's Functions (DFA3D/dfa3D/ops/multi_scale_3D_deform_attn.py);
the implementation lives in ``dfa3D.functional``."""
from ..functional import *  # noqa: F401,F403
from ..functional import __all__  # noqa: F401
