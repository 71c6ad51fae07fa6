"""Golden vectors (tests/golden/*.npz, float64, made by tests/golden/make_golden.py from the
grid_sample statement of the operator): the CPU checker must reproduce them, and so must the HIP
kernels."""
import glob
import os

import numpy as np
import pytest
import torch

GOLDEN = sorted(glob.glob(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "*.npz")))
TOL = dict(rtol=1e-10, atol=1e-11)


def _load(path):
    z = np.load(path, allow_pickle=False)
    return {k: torch.from_numpy(z[k]) for k in z.files}


def test_fixtures_present():
    assert len(GOLDEN) >= 3


@pytest.mark.parametrize("path", GOLDEN, ids=[os.path.basename(p)[:-4] for p in GOLDEN])
def test_checker_reproduces_golden(oracle, path):
    t = _load(path)
    out, score = oracle.dfa3d_forward(t["value"], t["dist"], t["shapes3"], t["lsi"], t["loc"], t["attn"])
    gv, gd, gl, ga = oracle.dfa3d_backward(t["value"], t["dist"], t["shapes3"], t["lsi"], t["loc"], t["attn"], score,
                                           t["grad_out"])
    for name, got in (("out", out), ("score", score), ("grad_value", gv), ("grad_dist", gd), ("grad_loc", gl),
                      ("grad_attn", ga)):
        torch.testing.assert_close(got, t[name], msg=lambda m, n=name: f"{n}: {m}", **TOL)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float64, torch.float32], ids=["f64", "f32"])
@pytest.mark.parametrize("path", GOLDEN, ids=[os.path.basename(p)[:-4] for p in GOLDEN])
def test_kernels_reproduce_golden(path, dtype):
    from dfa3D.functional import MultiScale3DDeformableAttnFunction
    t = _load(path)
    dev = torch.device("cuda:0")
    leaves = [t[k].to(dev, dtype).requires_grad_() for k in ("value", "dist", "loc", "attn")]
    out, score = MultiScale3DDeformableAttnFunction.apply(
        leaves[0], leaves[1], t["shapes3"].to(dev), t["lsi"].to(dev), leaves[2], leaves[3], 64)
    grads = torch.autograd.grad(out, leaves, t["grad_out"].to(dev, dtype))
    fwd = TOL if dtype == torch.float64 else dict(rtol=1e-5, atol=1e-5)
    bwd = TOL if dtype == torch.float64 else dict(rtol=1e-4, atol=1e-4)
    torch.testing.assert_close(out.detach().cpu().double(), t["out"], **fwd)
    torch.testing.assert_close(score.detach().cpu().double(), t["score"], **fwd)
    for g, name in zip(grads, ("grad_value", "grad_dist", "grad_loc", "grad_attn")):
        torch.testing.assert_close(g.cpu().double(), t[name], msg=lambda m, n=name: f"{n}: {m}", **bwd)
