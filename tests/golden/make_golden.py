"""Writes the golden vectors in this directory.

    python tests/golden/make_golden.py

The reference holds no golden vectors, known-answer tests or fixtures for this operator
(unittest_DFA3D.py is unseeded and only asserts "not NaN"), and its implementation is CUDA device
code that cannot be built or run in this image.  These vectors are therefore computed from the
textbook statement of the operator, in float64, by routines that share no code with the CPU checker
or the HIP kernels (tests/forms.py): output and every gradient from ``torch.nn.functional.grid_sample``
on the expanded volume value (x) dist with ``torch.autograd``, the depth scores from python loops over
the definition.  Both the CPU checker and the GPU kernels are tested against them.
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
from forms import SLOT_OF, brute_depth_score, tiny_case, volume_form  # noqa: E402

CASES = {
    # name: tiny_case arguments
    "two_levels_oob": dict(seed=101, B=2, M=2, C=3, D=5, Q=7, P=3, levels=((4, 6), (2, 3)), lo=-0.2, hi=1.2),
    "c32_four_levels": dict(seed=102, B=1, M=8, C=32, D=16, Q=6, P=8, levels=((6, 9), (4, 5), (3, 3), (2, 2)),
                            lo=-0.05, hi=1.05),
    "single_bin_depth": dict(seed=103, B=1, M=2, C=8, D=1, Q=5, P=2, levels=((5, 4),), lo=0.0, hi=1.0),
}


def main():
    for name, kw in CASES.items():
        t = tiny_case(**kw)
        leaves = [t[k].clone().requires_grad_() for k in ("value", "dist", "loc", "attn")]
        out = volume_form(leaves[0], leaves[1], t["levels"], leaves[2], leaves[3])
        gv, gd, gl, ga = torch.autograd.grad(out, leaves, t["grad_out"])
        score = torch.zeros(*t["loc"].shape[:-1], 4, dtype=torch.float64)
        for (b, q, m, l, p, dh, dw), s in brute_depth_score(t["dist"], t["levels"], t["lsi"], t["loc"]).items():
            score[b, q, m, l, p, SLOT_OF[(dh, dw)]] = s
        np.savez_compressed(
            os.path.join(HERE, name + ".npz"),
            value=t["value"].numpy(), dist=t["dist"].numpy(), loc=t["loc"].numpy(), attn=t["attn"].numpy(),
            shapes3=t["shapes3"].numpy(), lsi=t["lsi"].numpy(), grad_out=t["grad_out"].numpy(),
            out=out.detach().numpy(), score=score.numpy(), grad_value=gv.numpy(), grad_dist=gd.numpy(),
            grad_loc=gl.numpy(), grad_attn=ga.numpy())
        print(name, "points", score.numel() // 4)


if __name__ == "__main__":
    main()
