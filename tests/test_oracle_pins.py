"""Pins the CPU checker (oracle/) against statements of the operator it does not
share code with: the 5-D / 2-D grid_sample identities, brute-force loops from
the definition, closed forms, autograd through the grid_sample forms and finite
differences.  The reference ships no golden vectors for this path (its only
test, unittest_DFA3D.py:72-73, asserts "not NaN"), so these are what fix the
checker's results.  CPU only.
"""
import math

import pytest
import torch

import forms
from forms import SLOT_OF, brute_depth_score, brute_weighted_attention, msda_2d_form, tiny_case, volume_form

F64 = dict(rtol=1e-11, atol=1e-12)


@pytest.mark.parametrize("seed", [0, 1, 2, 3])
def test_forward_equals_volume_grid_sample(oracle, seed):
    t = tiny_case(seed)
    out, _ = oracle.dfa3d_forward(t["value"], t["dist"], t["shapes3"], t["lsi"], t["loc"], t["attn"])
    ref = volume_form(t["value"], t["dist"], t["levels"], t["loc"], t["attn"])
    torch.testing.assert_close(out, ref, **F64)


def test_forward_equals_volume_grid_sample_unnormalised_dist_single_bin(oracle):
    # D = 1 and unnormalised "distributions": every corner score is hd*dist or ld*dist of one bin
    t = tiny_case(5, D=1, normalise=False)
    out, _ = oracle.dfa3d_forward(t["value"], t["dist"], t["shapes3"], t["lsi"], t["loc"], t["attn"])
    ref = volume_form(t["value"], t["dist"], t["levels"], t["loc"], t["attn"])
    torch.testing.assert_close(out, ref, **F64)


def test_boundary_locations_match_volume_form(oracle):
    # locations exactly on pixel centres, map edges, and the skip thresholds
    t = tiny_case(7, Q=9, P=4)
    H, W = t["levels"][0]
    D = t["dist"].shape[-1]
    special = [0.0, 1.0, 0.5 / W, 1 - 0.5 / W, -0.5 / W, 1 + 0.5 / W, 0.5, 1.5 / W, -0.4999 / W]
    for i, s in enumerate(special):
        t["loc"][0, i, :, :, 0, 0] = s
        t["loc"][0, i, :, :, 1, 1] = s * W / H
        t["loc"][0, i, :, :, 2, 2] = s * W / D
        t["loc"][1, i, :, :, 3, :] = s
    out, _ = oracle.dfa3d_forward(t["value"], t["dist"], t["shapes3"], t["lsi"], t["loc"], t["attn"])
    ref = volume_form(t["value"], t["dist"], t["levels"], t["loc"], t["attn"])
    torch.testing.assert_close(out, ref, **F64)


@pytest.mark.parametrize("seed", [0, 4])
def test_depth_score_by_definition_and_slot_order(oracle, seed):
    t = tiny_case(seed, B=1, Q=5)
    score = oracle.depth_score_forward(t["dist"], t["shapes3"], t["lsi"], t["loc"])
    ref = brute_depth_score(t["dist"], t["levels"], t["lsi"], t["loc"])
    got = torch.empty_like(score)
    for (b, q, m, l, p, dh, dw), s in ref.items():
        got[b, q, m, l, p, SLOT_OF[(dh, dw)]] = s
    torch.testing.assert_close(score, got, **F64)
    assert (score != 0).any()


def test_depth_score_slots_name_their_pixels(oracle):
    # dist constant along depth and equal to a code of the pixel: with z strictly inside,
    # hd + ld = 1, so each slot returns the code of the pixel it was read from.
    H, W, D = 5, 7, 4
    code = (torch.arange(H).view(H, 1) * 100 + torch.arange(W).view(1, W)).double().view(1, H * W, 1, 1)
    dist = code.expand(1, H * W, 1, D).contiguous()
    shapes3 = torch.tensor([[H, W, D]])
    lsi = torch.tensor([0])
    loc = torch.tensor([(2.3 + 0.5) / W, (1.6 + 0.5) / H, 0.5], dtype=torch.float64).view(1, 1, 1, 1, 1, 3)
    s = oracle.depth_score_forward(dist, shapes3, lsi, loc).view(4)
    h0, w0 = 1, 2
    expect = [h0 * 100 + w0, h0 * 100 + w0 + 1, (h0 + 1) * 100 + w0 + 1, (h0 + 1) * 100 + w0]  # LT, RT, RB, LB
    torch.testing.assert_close(s, torch.tensor(expect, dtype=torch.float64), **F64)


def test_depth_score_closed_forms(oracle):
    H, W, D = 4, 4, 8
    shapes3, lsi = torch.tensor([[H, W, D]]), torch.tensor([0])
    xy = [0.55, 0.45]

    def run(dist, z):
        loc = torch.tensor(xy + [z], dtype=torch.float64).view(1, 1, 1, 1, 1, 3)
        return oracle.depth_score_forward(dist.contiguous(), shapes3, lsi, loc).view(4)

    uniform = torch.full((1, H * W, 1, D), 1.0 / D, dtype=torch.float64)
    torch.testing.assert_close(run(uniform, 0.37), torch.full((4,), 1.0 / D, dtype=torch.float64), **F64)
    k = 3
    onehot = torch.zeros(1, H * W, 1, D, dtype=torch.float64)
    onehot[..., k] = 1
    torch.testing.assert_close(run(onehot, (k + 0.5) / D), torch.ones(4).double(), **F64)
    torch.testing.assert_close(run(onehot, (k + 1.0) / D), torch.full((4,), 0.5, dtype=torch.float64), **F64)
    torch.testing.assert_close(run(onehot, (k + 1.5) / D), torch.zeros(4).double(), **F64)
    # below the first bin centre the low side is zero padding: score = ld * dist[0], ld = z*D + 0.5
    z = 0.2 / D
    torch.testing.assert_close(run(uniform, z), torch.full((4,), (z * D + 0.5) / D, dtype=torch.float64), **F64)
    # above the last bin centre: score = hd * dist[D-1], hd = 1 - (z*D - 0.5 - (D-1))
    z = 1 - 0.2 / D
    torch.testing.assert_close(run(uniform, z), torch.full((4,), (1 - (z * D - 0.5 - (D - 1))) / D, dtype=torch.float64), **F64)
    # depth outside (-1, D) in pixel units: point skipped
    assert run(uniform, -0.6 / D).abs().max() == 0 and run(uniform, 1 + 0.6 / D).abs().max() == 0
    # the score does not depend on where inside the pixel cell (x, y) falls
    a = oracle.depth_score_forward(onehot * 0.3 + uniform, shapes3, lsi,
                                   torch.tensor([0.51, 0.40, 0.5], dtype=torch.float64).view(1, 1, 1, 1, 1, 3))
    b = oracle.depth_score_forward(onehot * 0.3 + uniform, shapes3, lsi,
                                   torch.tensor([0.60, 0.49, 0.5], dtype=torch.float64).view(1, 1, 1, 1, 1, 3))
    torch.testing.assert_close(a, b, **F64)


def test_weighted_attention_with_unit_scores_is_plain_msda(oracle):
    t = tiny_case(11)
    ones = torch.ones(*t["loc"].shape[:-1], 4, dtype=torch.float64)
    loc2 = t["loc"][..., :2].contiguous()
    shapes2 = t["shapes3"][:, :2].contiguous()
    out = oracle.wms_forward(t["value"], shapes2, t["lsi"], loc2, t["attn"], ones)
    torch.testing.assert_close(out, msda_2d_form(t["value"], t["levels"], loc2, t["attn"]), **F64)
    # the (L,3)/(…,3) strided call is the same computation
    out3 = oracle.wms_forward(t["value"], t["shapes3"], t["lsi"], t["loc"], t["attn"], ones)
    assert torch.equal(out, out3)


def test_weighted_attention_arbitrary_scores_by_definition(oracle):
    t = tiny_case(12, B=1, Q=4)
    g = torch.Generator().manual_seed(99)
    score = torch.randn(*t["loc"].shape[:-1], 4, generator=g, dtype=torch.float64)
    out = oracle.wms_forward(t["value"], t["shapes3"], t["lsi"], t["loc"], t["attn"], score)
    ref = brute_weighted_attention(
        t["value"], t["levels"], t["lsi"], t["loc"], t["attn"],
        lambda b, q, m, l, p, dh, dw: float(score[b, q, m, l, p, SLOT_OF[(dh, dw)]]))
    torch.testing.assert_close(out, ref, **F64)


@pytest.mark.parametrize("seed", [0, 1, 2])
def test_one_stage_backward_equals_autograd_of_volume_form(oracle, seed):
    t = tiny_case(seed + 20)
    leaves = [t[k].clone().requires_grad_() for k in ("value", "dist", "loc", "attn")]
    ref_out = volume_form(leaves[0], leaves[1], t["levels"], leaves[2], leaves[3])
    gv, gd, gl, ga = torch.autograd.grad(ref_out, leaves, t["grad_out"])
    out, score = oracle.dfa3d_forward(t["value"], t["dist"], t["shapes3"], t["lsi"], t["loc"], t["attn"])
    ov, od, ol, oa = oracle.dfa3d_backward(t["value"], t["dist"], t["shapes3"], t["lsi"], t["loc"], t["attn"],
                                           score, t["grad_out"])
    tol = dict(rtol=1e-10, atol=1e-11)
    torch.testing.assert_close(ov, gv, **tol)
    torch.testing.assert_close(od, gd, **tol)
    torch.testing.assert_close(oa, ga, **tol)
    torch.testing.assert_close(ol, gl, **tol)
    assert gl[..., 2].abs().max() > 0 and gd.abs().max() > 0


def _central_difference(f, x, eps=1e-6):
    g = torch.zeros_like(x)
    flat, gf = x.view(-1), g.view(-1)
    for i in range(flat.numel()):
        old = flat[i].item()
        flat[i] = old + eps
        up = f()
        flat[i] = old - eps
        dn = f()
        flat[i] = old
        gf[i] = (up - dn) / (2 * eps)
    return g


def test_stage2_backward_by_finite_differences(oracle):
    # keeps locations away from pixel-cell borders, where the function has kinks
    t = tiny_case(31, B=1, Q=2, P=2, C=2, lo=0.05, hi=0.95)
    for l, (H, W) in enumerate(t["levels"]):
        for ax, n in ((0, W), (1, H)):
            c = t["loc"][:, :, :, l, :, ax] * n - 0.5
            frac = c - c.floor()
            c = c.floor() + frac.clamp(0.1, 0.9)
            t["loc"][:, :, :, l, :, ax] = (c + 0.5) / n
    g = torch.Generator().manual_seed(5)
    score = torch.rand(*t["loc"].shape[:-1], 4, generator=g, dtype=torch.float64) + 0.1
    loc2 = t["loc"][..., :2].contiguous()
    shapes2 = t["shapes3"][:, :2].contiguous()
    go = t["grad_out"]

    def f():
        return (oracle.wms_forward(t["value"], shapes2, t["lsi"], loc2, t["attn"], score) * go).sum().item()

    gv, gl, ga, gs = oracle.wms_backward(t["value"], shapes2, t["lsi"], loc2, t["attn"], score, go)
    tol = dict(rtol=1e-6, atol=1e-7)
    torch.testing.assert_close(gs, _central_difference(f, score), **tol)
    torch.testing.assert_close(ga, _central_difference(f, t["attn"]), **tol)
    torch.testing.assert_close(gl, _central_difference(f, loc2), **tol)
    torch.testing.assert_close(gv, _central_difference(f, t["value"]), **tol)


def test_stage1_backward_by_finite_differences(oracle):
    t = tiny_case(32, B=1, Q=2, P=2, lo=0.05, hi=0.95)
    D = t["dist"].shape[-1]
    c = t["loc"][..., 2] * D - 0.5
    t["loc"][..., 2] = (c.floor() + (c - c.floor()).clamp(0.1, 0.9) + 0.5) / D
    g = torch.Generator().manual_seed(6)
    gsc = torch.randn(*t["loc"].shape[:-1], 4, generator=g, dtype=torch.float64)

    def f():
        return (oracle.depth_score_forward(t["dist"], t["shapes3"], t["lsi"], t["loc"]) * gsc).sum().item()

    gd, gl = oracle.depth_score_backward(t["dist"], t["shapes3"], t["lsi"], t["loc"], gsc)
    tol = dict(rtol=1e-6, atol=1e-7)
    torch.testing.assert_close(gd, _central_difference(f, t["dist"]), **tol)
    # z gradient by differences; x and y gradients are identically zero (scores are piecewise constant in x, y)
    zg = _central_difference(f, t["loc"])[..., 2]
    torch.testing.assert_close(gl[..., 2], zg, **tol)
    assert gl[..., :2].abs().max() == 0


def test_two_stage_chain_equals_one_stage(oracle):
    t = tiny_case(40)
    out1, score = oracle.dfa3d_forward(t["value"], t["dist"], t["shapes3"], t["lsi"], t["loc"], t["attn"])
    loc2 = t["loc"][..., :2].contiguous()
    shapes2 = t["shapes3"][:, :2].contiguous()
    out2 = oracle.wms_forward(t["value"], shapes2, t["lsi"], loc2, t["attn"], score)
    assert torch.equal(out1, out2)


def test_skipped_points_have_zero_gradients(oracle):
    t = tiny_case(41, B=1, Q=3)
    t["loc"][0, 0, :, :, :, 0] = -0.3      # x far outside: stage 2 skips
    t["loc"][0, 1, :, :, :, 2] = 1.4       # z far outside: stage 1 skips, scores are zero
    out, score = oracle.dfa3d_forward(t["value"], t["dist"], t["shapes3"], t["lsi"], t["loc"], t["attn"])
    assert out[0, :2].abs().max() == 0 and score[0, :2].abs().max() == 0
    gv, gd, gl, ga = oracle.dfa3d_backward(t["value"], t["dist"], t["shapes3"], t["lsi"], t["loc"], t["attn"],
                                           score, t["grad_out"])
    assert gl[0, :2].abs().max() == 0 and ga[0, :2].abs().max() == 0
    assert gl[0, 2].abs().max() > 0


def test_float_path_tracks_double_path(oracle):
    t = tiny_case(50, B=2, Q=40, C=8, D=9, levels=((9, 11), (5, 6), (3, 3)), lo=-0.05, hi=1.05)
    f32 = {k: (v.float() if torch.is_tensor(v) and v.is_floating_point() else v) for k, v in t.items()}
    d64 = {k: (v.double() if torch.is_tensor(v) and v.is_floating_point() else v) for k, v in f32.items()}
    o32, s32 = oracle.dfa3d_forward(f32["value"], f32["dist"], f32["shapes3"], f32["lsi"], f32["loc"], f32["attn"])
    o64, s64 = oracle.dfa3d_forward(d64["value"], d64["dist"], d64["shapes3"], d64["lsi"], d64["loc"], d64["attn"])
    torch.testing.assert_close(o32.double(), o64, rtol=1e-5, atol=1e-5)
    g32 = oracle.dfa3d_backward(f32["value"], f32["dist"], f32["shapes3"], f32["lsi"], f32["loc"], f32["attn"],
                                s32, f32["grad_out"])
    g64 = oracle.dfa3d_backward(d64["value"], d64["dist"], d64["shapes3"], d64["lsi"], d64["loc"], d64["attn"],
                                s64, d64["grad_out"])
    for a, b in zip(g32, g64):
        torch.testing.assert_close(a.double(), b, rtol=1e-4, atol=1e-4)


def test_double_coordinates_are_floored_in_single_precision(oracle):
    # The reference calls floorf() on every scalar type
    # (ms_depth_score_sample_cuda_kernel.cuh:30-32), so a double pixel coordinate that rounds up
    # to an integer in float lands in the upper cell with a tiny negative fraction.
    H, W, D = 4, 8, 4
    code = torch.arange(H * W).double().view(1, H * W, 1, 1).expand(1, H * W, 1, D).contiguous()
    shapes3, lsi = torch.tensor([[H, W, D]]), torch.tensor([0])
    x_pix = 3.0 - 1e-12                       # floor() in double = 2, floorf(float(x)) = 3
    loc = torch.tensor([(x_pix + 0.5) / W, (1.25 + 0.5) / H, 0.5], dtype=torch.float64).view(1, 1, 1, 1, 1, 3)
    w_im = float(loc[0, 0, 0, 0, 0, 0]) * W - 0.5
    assert math.floor(w_im) == 2 and math.floor(float(torch.tensor(w_im).float())) == 3
    s = oracle.depth_score_forward(code, shapes3, lsi, loc).view(4)
    assert s[0].item() == 1 * W + 3 and s[1].item() == 1 * W + 4


def test_thread_count_does_not_change_results(oracle):
    t = tiny_case(60, B=3, Q=11)
    prev = oracle.set_threads(1)
    try:
        a = oracle.dfa3d_forward(t["value"], t["dist"], t["shapes3"], t["lsi"], t["loc"], t["attn"])
        ga = oracle.dfa3d_backward(t["value"], t["dist"], t["shapes3"], t["lsi"], t["loc"], t["attn"], a[1], t["grad_out"])
        oracle.set_threads(4)
        b = oracle.dfa3d_forward(t["value"], t["dist"], t["shapes3"], t["lsi"], t["loc"], t["attn"])
        gb = oracle.dfa3d_backward(t["value"], t["dist"], t["shapes3"], t["lsi"], t["loc"], t["attn"], b[1], t["grad_out"])
    finally:
        oracle.set_threads(prev)
    for x, y in zip(a + ga, b + gb):
        assert torch.equal(x, y)


def test_float_geometry_instantiation_tracks_both_precisions(oracle):
    """The third instantiation of the checker (float64 arithmetic on the float32 path's pixel coordinates, the
    yardstick for float32 summation error in the GPU tests) is the same code as the other two: on float32
    inputs it agrees with the float64 instantiation up to what a float32 pixel coordinate is worth, and with
    the float32 instantiation up to float32 rounding of the sums."""
    t = tiny_case(77, B=2, C=8, M=3, Q=40, P=4, D=6, levels=((90, 120), (7, 9)), dtype=torch.float32)
    args32 = (t["value"], t["dist"], t["shapes3"], t["lsi"], t["loc"], t["attn"])
    args64 = tuple(a.double() if a.is_floating_point() else a for a in args32)

    def run(args, go):
        out, score = oracle.dfa3d_forward(*args)
        return (out, score) + tuple(oracle.dfa3d_backward(*args, score, go))

    r32 = run(args32, t["grad_out"])
    r64 = run(args64, t["grad_out"].double())
    with oracle.float_geometry():
        rg = run(args64, t["grad_out"].double())
    for a, b, c in zip(r32, r64, rg):
        assert c.dtype == torch.float64
        torch.testing.assert_close(c, b, rtol=1e-4, atol=1e-4)                 # coordinates differ by <= 120 * 2^-24
        torch.testing.assert_close(c, a.double(), rtol=1e-5, atol=2e-6)        # sums differ by float32 rounding
    assert not torch.equal(rg[2], r64[2])                                      # and it is not the plain float64 path
