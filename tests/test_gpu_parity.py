"""GPU parity: the HIP kernels, called through the autograd Functions (and so through the C ABI),
against the CPU checker on identical seeded inputs.

Tolerances (stated by the task): fp32 forward rtol = atol = 1e-5; fp32 backward rtol = atol = 1e-4
(floating-point atomics make the summation order of grad_value / grad_dist nondeterministic);
fp64 1e-10 / 1e-11 forward / backward; bf16 storage: see test_bf16_storage.
"""
import pytest
import torch

from forms import tiny_case

pytestmark = pytest.mark.gpu

F32_FWD = dict(rtol=1e-5, atol=1e-5)
F32_BWD = dict(rtol=1e-4, atol=1e-4)


def _dev():
    assert torch.cuda.is_available(), "these tests need the MI355X"
    return torch.device("cuda:0")


def _functions():
    from dfa3D.ops.multi_scale_3D_deform_attn import (MultiScale3DDeformableAttnFunction,
                                                      MultiScaleDepthScoreSampleFunction,
                                                      WeightedMultiScaleDeformableAttnFunction)
    return MultiScale3DDeformableAttnFunction, MultiScaleDepthScoreSampleFunction, \
        WeightedMultiScaleDeformableAttnFunction


def _gpu_one_stage(inp, dev, grad_score=None):
    F1, _, _ = _functions()
    value = inp["value"].to(dev).requires_grad_()
    dist = inp["value_dpt_dist"].to(dev).requires_grad_()
    loc = inp["sampling_locations"].to(dev).requires_grad_()
    attn = inp["attention_weights"].to(dev).requires_grad_()
    out, score = F1.apply(value, dist, inp["spatial_shapes"].to(dev), inp["level_start_index"].to(dev), loc, attn, 64)
    outs, gouts = [out], [inp["grad_output"].to(dev)]
    if grad_score is not None:
        outs.append(score)
        gouts.append(grad_score.to(dev))
    gv, gd, gl, ga = torch.autograd.grad(outs, [value, dist, loc, attn], gouts)
    torch.cuda.synchronize()
    return out.detach().cpu(), score.detach().cpu(), gv.cpu(), gd.cpu(), gl.cpu(), ga.cpu()


def _oracle_one_stage(oracle, inp):
    out, score = oracle.dfa3d_forward(inp["value"], inp["value_dpt_dist"], inp["spatial_shapes"],
                                      inp["level_start_index"], inp["sampling_locations"], inp["attention_weights"])
    gv, gd, gl, ga = oracle.dfa3d_backward(inp["value"], inp["value_dpt_dist"], inp["spatial_shapes"],
                                           inp["level_start_index"], inp["sampling_locations"],
                                           inp["attention_weights"], score, inp["grad_output"])
    return out, score, gv, gd, gl, ga


def _as_inputs(t):
    return {"value": t["value"], "value_dpt_dist": t["dist"], "spatial_shapes": t["shapes3"],
            "level_start_index": t["lsi"], "sampling_locations": t["loc"], "attention_weights": t["attn"],
            "grad_output": t["grad_out"]}


def _compare(got, want, fwd_tol, bwd_tol):
    names = ["output", "depth_score", "grad_value", "grad_dist", "grad_loc", "grad_attn"]
    for i, (g, w, n) in enumerate(zip(got, want, names)):
        tol = fwd_tol if i < 2 else bwd_tol
        torch.testing.assert_close(g, w, msg=lambda m, n=n: f"{n}: {m}", **tol)


def _corner_hits(inp):
    """Number of (sampling point, corner) pairs that land on each key, (B, S, M): the number of terms summed
    into that key's grad_value row (twice that, at most, into each of its grad_dist bins)."""
    loc = inp["sampling_locations"].float()
    B, Q, M, L, P, _ = loc.shape
    shapes, lsi = inp["spatial_shapes"], inp["level_start_index"]
    S = inp["value"].shape[1]
    hits = torch.zeros(B * S * M, dtype=torch.int64)
    b = torch.arange(B).view(B, 1, 1, 1).expand(B, Q, M, P)
    m = torch.arange(M).view(1, 1, M, 1).expand(B, Q, M, P)
    for l in range(L):
        H, W = int(shapes[l, 0]), int(shapes[l, 1])
        w_im, h_im = loc[:, :, :, l, :, 0] * W - 0.5, loc[:, :, :, l, :, 1] * H - 0.5     # separately rounded, as the kernels do
        inside = (h_im > -1) & (w_im > -1) & (h_im < H) & (w_im < W)
        h0, w0 = torch.floor(h_im).long(), torch.floor(w_im).long()
        for dh in (0, 1):
            for dw in (0, 1):
                hc, wc = h0 + dh, w0 + dw
                ok = inside & (hc >= 0) & (hc < H) & (wc >= 0) & (wc < W)
                key = int(lsi[l]) + hc * W + wc
                hits += torch.bincount(((b * S + key) * M + m)[ok], minlength=B * S * M)
    return hits.view(B, S, M)


def _sum_truth(oracle, inp):
    """Float64 checker on the float32 inputs: exact grad_value / grad_dist, the sums of the absolute values of
    their terms (checker run on |value| and |grad_output|; weights and distributions are non-negative) and
    the number of corner hits per key.  The float64 run takes the float32 path's pixel coordinates
    (oracle.float_geometry: a float32 coordinate of up to 200 pixels is itself only good to 1e-5 of a pixel, which
    is a property of the inputs' type, not of the summation that is being checked)."""
    assert inp["attention_weights"].min() >= 0 and inp["value_dpt_dist"].min() >= 0
    f64 = {k: (v.double() if v.is_floating_point() else v) for k, v in inp.items()}
    args = [f64[k] for k in ("value", "value_dpt_dist", "spatial_shapes", "level_start_index", "sampling_locations",
                             "attention_weights")]
    with oracle.float_geometry():
        _, score = oracle.dfa3d_forward(*args)
        t_gv, t_gd, _, _ = oracle.dfa3d_backward(*args, score, f64["grad_output"])
        args[0] = args[0].abs()
        a_gv, a_gd, _, _ = oracle.dfa3d_backward(*args, score, f64["grad_output"].abs())
    return dict(gv=t_gv, gd=t_gd, abs_gv=a_gv, abs_gd=a_gd, hits=_corner_hits(inp).double().unsqueeze(-1))


def _assert_sums_within_term_count_bound(oracle, inp, gv, gd, storage_rel=0.0, term_rel=0.0, shared_dist=False,
                                         atomic_rel=0.0):
    """grad_value / grad_dist of the kernels against the FLOAT64 checker on the same inputs.
    An element that is a float32 sum of n terms t_i, formed in any order from terms that each carry a few
    roundings (a dot product over C channels for grad_dist), is within (n + extra) * 2^-24 * sum|t_i| of the
    exact sum.  No relative slack is added for float32 results.  `storage_rel` is the rounding of results that
    are stored in a shorter type (2^-8 for bfloat16: the sums themselves are float32 in every mode), `term_rel`
    the rounding of every TERM where an intermediate tensor is stored in bfloat16 between two kernels.
    `shared_dist`: grad_dist is summed over the heads (one distribution for all heads); `inp` then holds the
    distribution repeated per head.  `atomic_rel`: gradients stored in bfloat16 by the kernel itself: the rows
    several tiles share (and bins split over several work items) are added with packed bfloat16 atomics, k adds
    that each round the stored sum, k * 2^-9 of the largest partial sum at worst."""
    t = _sum_truth(oracle, inp)
    n, C, u = t["hits"], inp["value"].shape[3], 2.0 ** -24
    bound_gv = ((n + 16) * u + term_rel + atomic_rel) * t["abs_gv"] + 1e-30
    bound_gd = ((2 * n + C + 16) * u + term_rel + atomic_rel) * t["abs_gd"] + 1e-30
    t_gd = t["gd"]
    if shared_dist:
        M = t_gd.shape[2]
        t_gd, bound_gd = t_gd.sum(2, keepdim=True), bound_gd.sum(2, keepdim=True) + M * u * t["abs_gd"].sum(2, keepdim=True)
    for name, got, truth, bound in (("grad_value", gv, t["gv"], bound_gv), ("grad_dist", gd, t_gd, bound_gd)):
        err = (got.double() - truth).abs()
        worst = (err / (bound + storage_rel * truth.abs())).max().item()
        assert worst <= 1.0, f"{name}: error is {worst:.3g} x the term-count bound (max |err| {err.max().item():.3g})"
        # and as a whole the tensor is far inside the backward tolerance
        rel = (err.pow(2).sum() / truth.pow(2).sum().clamp(min=1e-300)).sqrt().item()
        assert rel <= max(1e-5, storage_rel, 4 * term_rel), f"{name}: relative RMS error {rel:.3g}"


def _per_point_truth(oracle, inp):
    """Float64 checker on the float32 path's pixel coordinates for the four per-point / per-unit tensors (output,
    depth_score, grad_loc, grad_attn), and for each of them the sum of the absolute values of the terms the float32
    path adds up, obtained from the checker alone:
      output      forward on |value| (bilinear weights, scores and attention weights are non-negative)
      depth_score the score itself (two non-negative terms)
      grad_attn   backward on |value|, |grad_output|
      grad_loc x  W a (hh (s1 - s0) + lh (s2 - s3)), s_k = score_k dot_k: stage-2 backward on |value|, |grad_output|
                  with the scores of the subtracted corners (LT, LB) set to zero, minus the same with the scores of
                  the added corners (RT, RB) set to zero; y likewise with (RB, LB) against (LT, RT)
      grad_loc z  Dd sum_k gs_k (hi_k - lo_k): Dd sum_k |gs_k| (hi_k + lo_k), |gs_k| from that stage-2 backward, the
                  two taps of every corner from stage-1 forwards at the centres of bins d0 and d0 + 1."""
    assert inp["attention_weights"].min() >= 0 and inp["value_dpt_dist"].min() >= 0
    f64 = {k: (v.double() if v.is_floating_point() else v) for k, v in inp.items()}
    v, d, sh, lsi, loc, a, go = (f64[k] for k in ("value", "value_dpt_dist", "spatial_shapes", "level_start_index",
                                                  "sampling_locations", "attention_weights", "grad_output"))
    with oracle.float_geometry():
        out, score = oracle.dfa3d_forward(v, d, sh, lsi, loc, a)
        _, _, gl, ga = oracle.dfa3d_backward(v, d, sh, lsi, loc, a, score, go)
        abs_out = oracle.wms_forward(v.abs(), sh, lsi, loc, a, score)
        _, _, abs_ga, abs_gs = oracle.wms_backward(v.abs(), sh, lsi, loc, a, score, go.abs())

        def masked(keep):
            sc = score * torch.tensor(keep, dtype=score.dtype)
            return oracle.wms_backward(v.abs(), sh, lsi, loc, a, sc.contiguous(), go.abs())[1]
        abs_x = masked([0., 1., 1., 0.])[..., 0] - masked([1., 0., 0., 1.])[..., 0]       # slots LT, RT, RB, LB
        abs_y = masked([0., 0., 1., 1.])[..., 1] - masked([1., 1., 0., 0.])[..., 1]
        # the two depth taps of every corner: scores at the centres of the bins below and above the location
        Dd = sh[:, 2].double().view(1, 1, 1, -1, 1)
        d_im = (loc[..., 2].float() * Dd.float() - 0.5).double()                         # the float32 path's coordinate
        d0 = torch.floor(d_im)
        taps = 0
        for shift in (0.5, 1.5):
            at = loc.clone()
            at[..., 2] = ((d0 + shift) / Dd).float().double()
            taps = taps + oracle.depth_score_forward(d, sh, lsi, at.contiguous())
        abs_z = Dd * (abs_gs * taps).sum(-1)
    abs_gl = torch.stack([abs_x, abs_y, abs_z], -1)
    return dict(out=out, score=score, gl=gl, ga=ga, abs_out=abs_out, abs_score=score.abs(), abs_gl=abs_gl, abs_ga=abs_ga)


def _assert_per_point_within_term_count_bound(oracle, inp, out, score, gl, ga, term_rel=0.0, storage_rel=0.0):
    """output, depth_score, grad_loc and grad_attn of the kernels against the float64 checker, each element within
    (n + extra) * 2^-24 * sum|t_i| of the exact value, n the number of terms of its sum: 4 L P corner rows for an
    output element, 2 taps for a score, C channels per dot product and four corners for the per-point gradients
    (the z gradient chains two such sums).  `term_rel`: relative rounding every term carries where an intermediate
    tensor is stored in bfloat16 between two kernels; `storage_rel`: rounding of the result itself (bfloat16
    outputs).  The checker takes the float32 path's pixel coordinates, so the rounding of loc * size - 0.5 is no
    part of the difference."""
    t = _per_point_truth(oracle, inp)
    u = 2.0 ** -24
    C = inp["value"].shape[3]
    LP = inp["sampling_locations"].shape[3] * inp["sampling_locations"].shape[4]
    checks = (("output", out, t["out"], (4 * LP + 16) * u, t["abs_out"]),
              ("depth_score", score, t["score"], 12 * u, t["abs_score"]),
              ("grad_loc", gl, t["gl"], (2 * C + 48) * u, t["abs_gl"]),
              ("grad_attn", ga, t["ga"], (C + 24) * u, t["abs_ga"]))
    for name, got, truth, rel, abs_sum in checks:
        err = (got.double() - truth).abs()
        bound = (rel + term_rel) * abs_sum + storage_rel * truth.abs() + 1e-30
        worst = (err / bound).max().item()
        assert worst <= 1.0, f"{name}: error is {worst:.3g} x the term-count bound (max |err| {err.max().item():.3g})"


TINY = [
    dict(seed=0),                                                    # C=3 (generic row tiling), L*P=6
    dict(seed=1, C=32, M=8, Q=5, P=8, levels=((6, 9), (4, 5), (3, 3), (2, 2))),   # L*P=32, C=32 fast path
    dict(seed=2, C=64, M=4, Q=3, P=4, levels=((5, 5),)),             # single level, C=64
    dict(seed=3, C=16, M=3, Q=2, P=30, levels=((4, 6), (2, 3), (3, 2))),          # L*P=90 > 64: chunked units
    dict(seed=4, C=5, M=1, Q=9, P=1, levels=((3, 4),)),              # L*P=1
    dict(seed=5, C=128, M=2, Q=2, P=2, levels=((4, 4), (2, 2)), D=1),             # D=1
    dict(seed=6, C=100, M=2, Q=3, P=3, levels=((4, 4), (2, 3))),     # C not a power of two, > 64: two passes
    dict(seed=7, C=256, M=1, Q=2, P=2, levels=((3, 3),)),
]


@pytest.mark.parametrize("case", TINY, ids=lambda c: "-".join(f"{k}{v}" for k, v in c.items() if k != "levels"))
def test_fp64_one_stage_matches_checker(oracle, case):
    dev = _dev()
    inp = _as_inputs(tiny_case(**case))
    got = _gpu_one_stage(inp, dev)
    want = _oracle_one_stage(oracle, inp)
    _compare(got, want, dict(rtol=1e-10, atol=1e-11), dict(rtol=1e-10, atol=1e-11))


FP32_EXTRA = [
    dict(seed=8, C=48, M=12, Q=11, P=3, D=10, levels=((9, 7), (5, 4), (2, 3))),   # 12 heads: two heads per XCD class
    dict(seed=9, C=64, M=16, Q=40, P=4, D=6, levels=((20, 31), (10, 16))),        # C=64: eight channels per lane
    dict(seed=10, C=32, M=5, Q=300, P=8, D=64, levels=((33, 47), (17, 24), (9, 12), (5, 6))),   # several tiles per level
]


def _random_case(seed):
    """A shape drawn from a seeded generator: odd channel counts, head counts that are no multiple of the
    eight XCD classes, one to five levels of unrelated sizes (maps smaller than a tile, maps of many tiles)."""
    import random
    r = random.Random(seed)
    L = r.randint(1, 5)
    levels = tuple((r.randint(1, 40), r.randint(1, 40)) for _ in range(L))
    return dict(seed=seed, B=r.randint(1, 3), M=r.choice([1, 2, 3, 4, 6, 8, 9, 16]),
                C=r.choice([1, 4, 8, 12, 16, 24, 32, 40, 64, 72, 128]), D=r.choice([1, 2, 3, 8, 17, 32, 64, 80]),
                Q=r.randint(1, 400), P=r.randint(1, 9), levels=levels, lo=r.choice([0.0, -0.2]), hi=r.choice([1.0, 1.2]))


@pytest.mark.parametrize("seed", range(100, 124))
def test_fp32_random_shapes_match_checker(oracle, seed):
    dev = _dev()
    case = _random_case(seed)
    print("case", case, flush=True)
    t = tiny_case(**case)
    inp = {k: (v.float() if v.is_floating_point() else v) for k, v in _as_inputs(t).items()}
    _compare(_gpu_one_stage(inp, dev), _oracle_one_stage(oracle, inp), F32_FWD, F32_BWD)


@pytest.mark.parametrize("case", TINY + FP32_EXTRA, ids=lambda c: f"seed{c['seed']}")
def test_fp32_one_stage_matches_checker_tiny(oracle, case):
    dev = _dev()
    t = tiny_case(**case)
    inp = {k: (v.float() if v.is_floating_point() else v) for k, v in _as_inputs(t).items()}
    _compare(_gpu_one_stage(inp, dev), _oracle_one_stage(oracle, inp), F32_FWD, F32_BWD)


def test_fp64_two_stage_matches_checker_and_chains(oracle):
    dev = _dev()
    _, F3, F2 = _functions()
    t = tiny_case(11, C=32, M=4, Q=6, P=4, levels=((5, 7), (3, 4)))
    inp = _as_inputs(t)
    dist = inp["value_dpt_dist"].to(dev).requires_grad_()
    value = inp["value"].to(dev).requires_grad_()
    loc3 = inp["sampling_locations"].to(dev).requires_grad_()
    attn = inp["attention_weights"].to(dev).requires_grad_()
    shapes3, lsi = inp["spatial_shapes"].to(dev), inp["level_start_index"].to(dev)
    score = F3.apply(dist, shapes3, lsi, loc3, 64)
    out = F2.apply(value, shapes3[:, :2].contiguous(), lsi, loc3[..., :2].contiguous(), attn, score, 64)
    gv, gd, gl, ga = torch.autograd.grad(out, [value, dist, loc3, attn], inp["grad_output"].to(dev))
    want = _oracle_one_stage(oracle, inp)
    got = (out.detach().cpu(), score.detach().cpu(), gv.cpu(), gd.cpu(), gl.cpu(), ga.cpu())
    _compare(got, want, dict(rtol=1e-10, atol=1e-11), dict(rtol=1e-10, atol=1e-11))


def test_fp64_stage2_alone_arbitrary_scores(oracle):
    dev = _dev()
    _, _, F2 = _functions()
    t = tiny_case(12, C=32, M=2, Q=4, P=4, levels=((5, 7), (3, 4)))
    g = torch.Generator().manual_seed(3)
    score = torch.randn(*t["loc"].shape[:-1], 4, generator=g, dtype=torch.float64)
    shapes2 = t["shapes3"][:, :2].contiguous()
    loc2 = t["loc"][..., :2].contiguous()
    leaves = [x.to(dev).requires_grad_() for x in (t["value"], loc2, t["attn"], score)]
    out = F2.apply(leaves[0], shapes2.to(dev), t["lsi"].to(dev), leaves[1], leaves[2], leaves[3], 64)
    gv, gl, ga, gs = torch.autograd.grad(out, leaves, t["grad_out"].to(dev))
    o_out = oracle.wms_forward(t["value"], shapes2, t["lsi"], loc2, t["attn"], score)
    o_gv, o_gl, o_ga, o_gs = oracle.wms_backward(t["value"], shapes2, t["lsi"], loc2, t["attn"], score, t["grad_out"])
    tol = dict(rtol=1e-10, atol=1e-11)
    for a, b in ((out, o_out), (gv, o_gv), (gl, o_gl), (ga, o_ga), (gs, o_gs)):
        torch.testing.assert_close(a.detach().cpu(), b, **tol)


def test_fp64_stage1_alone_backward(oracle):
    dev = _dev()
    _, F3, _ = _functions()
    t = tiny_case(13, M=3, Q=6, P=5, D=7, levels=((5, 7), (3, 4)))
    g = torch.Generator().manual_seed(4)
    gsc = torch.randn(*t["loc"].shape[:-1], 4, generator=g, dtype=torch.float64)
    dist = t["dist"].to(dev).requires_grad_()
    loc = t["loc"].to(dev).requires_grad_()
    score = F3.apply(dist, t["shapes3"].to(dev), t["lsi"].to(dev), loc, 64)
    gd, gl = torch.autograd.grad(score, [dist, loc], gsc.to(dev))
    o_gd, o_gl = oracle.depth_score_backward(t["dist"], t["shapes3"], t["lsi"], t["loc"], gsc)
    tol = dict(rtol=1e-10, atol=1e-11)
    torch.testing.assert_close(score.detach().cpu(), oracle.depth_score_forward(t["dist"], t["shapes3"], t["lsi"], t["loc"]), **tol)
    torch.testing.assert_close(gd.cpu(), o_gd, **tol)
    torch.testing.assert_close(gl.cpu(), o_gl, **tol)
    assert gl[..., :2].abs().max().item() == 0


def test_gradient_through_depth_score_output(oracle):
    """A gradient arriving at the depth_score output is chained (the reference refuses it)."""
    dev = _dev()
    t = tiny_case(14, C=32, M=2, Q=4, P=4, levels=((5, 7), (3, 4)))
    inp = _as_inputs(t)
    g = torch.Generator().manual_seed(8)
    gsc = torch.randn(*t["loc"].shape[:-1], 4, generator=g, dtype=torch.float64)
    got = _gpu_one_stage(inp, dev, grad_score=gsc)
    want = list(_oracle_one_stage(oracle, inp))
    extra_gd, extra_gl = oracle.depth_score_backward(t["dist"], t["shapes3"], t["lsi"], t["loc"], gsc)
    want[3] = want[3] + extra_gd
    want[4] = want[4] + extra_gl
    _compare(got, want, dict(rtol=1e-10, atol=1e-11), dict(rtol=1e-10, atol=1e-11))


@pytest.mark.parametrize("dtype", [torch.float64, torch.float32], ids=["fp64", "fp32"])
@pytest.mark.parametrize("width", [2, 3])
def test_plain_deformable_attention_matches_grid_sample(oracle, dtype, width):
    """MultiScaleDeformableAttnFunction (no depth scores) against multi-scale deformable attention written
    with 2-D grid_sample and differentiated by autograd, and against the checker's stage 2 with scores of 1."""
    from forms import msda_2d_form
    from dfa3D.functional import MultiScaleDeformableAttnFunction
    dev = _dev()
    t = tiny_case(21, C=32, M=4, Q=9, P=4, levels=((6, 9), (4, 5), (3, 3)), dtype=dtype)
    shapes = t["shapes3"][:, :width].contiguous()
    loc = t["loc"][..., :width].contiguous()
    cpu = [x.clone().requires_grad_() for x in (t["value"], loc, t["attn"])]
    want = msda_2d_form(cpu[0], t["levels"], cpu[1][..., :2], cpu[2])
    want_grads = torch.autograd.grad(want, cpu, t["grad_out"])
    gpu = [x.to(dev).requires_grad_() for x in (t["value"], loc, t["attn"])]
    out = MultiScaleDeformableAttnFunction.apply(gpu[0], shapes.to(dev), t["lsi"].to(dev), gpu[1], gpu[2], 64)
    grads = torch.autograd.grad(out, gpu, t["grad_out"].to(dev))
    fwd_tol, bwd_tol = (dict(rtol=1e-10, atol=1e-11),) * 2 if dtype == torch.float64 else (F32_FWD, F32_BWD)
    torch.testing.assert_close(out.detach().cpu(), want.detach(), **fwd_tol)
    for g, w in zip(grads, want_grads):
        torch.testing.assert_close(g.cpu(), w, **bwd_tol)
    ones = torch.ones(*t["attn"].shape, 4, dtype=dtype)
    torch.testing.assert_close(out.detach().cpu(), oracle.wms_forward(
        t["value"], t["shapes3"][:, :2].contiguous(), t["lsi"], t["loc"][..., :2].contiguous(), t["attn"], ones), **fwd_tol)


def _shared_dist_expectation(oracle, inp, grad_wu=None):
    """Checker results for a distribution shared by the heads: the checker sees the 8-fold repeat the
    reference's caller makes (spatial_cross_attention.py:496-497) and its grad_dist is summed over heads;
    a gradient at the weight_update output enters as a gradient of the scores and of the weights."""
    M = inp["value"].shape[2]
    rep = dict(inp)
    rep["value_dpt_dist"] = inp["value_dpt_dist"].repeat(1, 1, M // inp["value_dpt_dist"].shape[2], 1).contiguous()
    out, score, gv, gd, gl, ga = _oracle_one_stage(oracle, rep)
    attn = inp["attention_weights"]
    wu = (score.mean(-1) * attn).flatten(-2).sum(-1, keepdim=True)
    if grad_wu is not None:
        gsc = (grad_wu[..., None, None] * attn[..., None] / 4).expand_as(score).contiguous()
        extra_gd, extra_gl = oracle.depth_score_backward(rep["value_dpt_dist"], inp["spatial_shapes"],
                                                         inp["level_start_index"], inp["sampling_locations"], gsc)
        gd = gd + extra_gd
        gl = gl + extra_gl
        ga = ga + grad_wu[..., None] * score.mean(-1)
    if inp["value_dpt_dist"].shape[2] == 1:
        gd = gd.sum(2, keepdim=True)
    return out, score, wu, gv, gd, gl, ga


@pytest.mark.parametrize("case", [TINY[0], TINY[1], TINY[3], TINY[4]], ids=lambda c: f"seed{c['seed']}")
@pytest.mark.parametrize("dtype", [torch.float64, torch.float32], ids=["fp64", "fp32"])
def test_shared_distribution_and_weight_update(oracle, case, dtype):
    """dist (B,S,1,D) used by every head, with the score tensor and with the fused weight_update output
    (gradients arriving at both outputs), against the checker on the repeated distribution.  fp64 runs the
    kernels with device-memory atomics, fp32 the LDS-tile kernels."""
    from dfa3D.functional import MultiScale3DDeformableAttnFunction, MultiScale3DDeformableAttnWeightUpdateFunction
    dev = _dev()
    t = tiny_case(**case)
    inp = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in _as_inputs(t).items()}
    inp["value_dpt_dist"] = inp["value_dpt_dist"][:, :, :1].contiguous()
    g = torch.Generator().manual_seed(77)
    grad_wu = torch.randn(*inp["attention_weights"].shape[:3], 1, generator=g, dtype=dtype)
    fwd_tol, bwd_tol = (dict(rtol=1e-10, atol=1e-11),) * 2 if dtype == torch.float64 else (F32_FWD, F32_BWD)

    def leaves():
        return [inp[k].to(dev).requires_grad_() for k in ("value", "value_dpt_dist", "sampling_locations",
                                                          "attention_weights")]
    shapes3, lsi, go = inp["spatial_shapes"].to(dev), inp["level_start_index"].to(dev), inp["grad_output"].to(dev)

    # (output, depth_score) with the shared distribution
    want = _shared_dist_expectation(oracle, inp)
    v, d, loc, a = leaves()
    out, score = MultiScale3DDeformableAttnFunction.apply(v, d, shapes3, lsi, loc, a, 64)
    grads = torch.autograd.grad(out, [v, d, loc, a], go)
    got = [x.detach().cpu() for x in (out, score, *grads)]
    _compare(got, [want[0], want[1], *want[3:]], fwd_tol, bwd_tol)

    # (output, weight_update), gradients at both
    want = _shared_dist_expectation(oracle, inp, grad_wu=grad_wu)
    v, d, loc, a = leaves()
    out, wu = MultiScale3DDeformableAttnWeightUpdateFunction.apply(v, d, shapes3, lsi, loc, a, 64)
    grads = torch.autograd.grad([out, wu], [v, d, loc, a], [go, grad_wu.to(dev)])
    torch.testing.assert_close(wu.detach().cpu(), want[2], **fwd_tol)
    got = [x.detach().cpu() for x in (out, score, *grads)]
    _compare(got, [want[0], want[1], *want[3:]], fwd_tol, bwd_tol)

    # weight_update with a distribution per head, gradient at weight_update alone
    inp_m = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in _as_inputs(t).items()}
    want = _shared_dist_expectation(oracle, inp_m, grad_wu=grad_wu)
    v, d, loc, a = [inp_m[k].to(dev).requires_grad_() for k in ("value", "value_dpt_dist", "sampling_locations",
                                                                 "attention_weights")]
    out, wu = MultiScale3DDeformableAttnWeightUpdateFunction.apply(v, d, shapes3, lsi, loc, a, 64)
    grads = torch.autograd.grad([out, wu], [v, d, loc, a], [go, grad_wu.to(dev)])
    torch.testing.assert_close(wu.detach().cpu(), want[2], **fwd_tol)
    _compare([out.detach().cpu(), want[1], *[x.cpu() for x in grads]], [want[0], want[1], *want[3:]], fwd_tol, bwd_tol)


def test_fp32_base_shape_shared_distribution_weight_update(oracle):
    """BEVFormer-base shape as its caller has it: one distribution for the 8 heads, weight_update wanted."""
    from dfa3D.functional import MultiScale3DDeformableAttnWeightUpdateFunction
    from dfa3D.workloads import WORKLOADS, make_inputs
    dev = _dev()
    inp = make_inputs(WORKLOADS["base"])
    inp["value_dpt_dist"] = inp["value_dpt_dist"][:, :, :1].contiguous()
    want = _shared_dist_expectation(oracle, inp)
    v, d, loc, a = [inp[k].to(dev).requires_grad_() for k in ("value", "value_dpt_dist", "sampling_locations",
                                                               "attention_weights")]
    out, wu = MultiScale3DDeformableAttnWeightUpdateFunction.apply(
        v, d, inp["spatial_shapes"].to(dev), inp["level_start_index"].to(dev), loc, a, 64)
    grads = torch.autograd.grad(out, [v, d, loc, a], inp["grad_output"].to(dev))
    torch.testing.assert_close(wu.detach().cpu(), want[2], **F32_FWD)
    _compare([out.detach().cpu(), want[1], *[x.cpu() for x in grads]], [want[0], want[1], *want[3:]], F32_FWD, F32_BWD)


@pytest.mark.parametrize("name", ["unit", "small"])
def test_fp32_workloads_match_checker(oracle, name):
    from dfa3D.workloads import WORKLOADS, make_inputs
    dev = _dev()
    inp = make_inputs(WORKLOADS[name])
    _compare(_gpu_one_stage(inp, dev), _oracle_one_stage(oracle, inp), F32_FWD, F32_BWD)


@pytest.mark.parametrize("Q", [2500, 999])
def test_fp32_model_like_locations_match_checker(oracle, Q):
    """Locations as a model produces them (queries in raster order over the image, the points of a query within a
    few pixels of each other): one query puts several points into the same tile and the same pixel, and the
    binning kernels spread each block's queries over the whole range (999 queries: not a multiple of anything)."""
    from dfa3D.workloads import WORKLOADS, make_inputs, scaled
    dev = _dev()
    inp = make_inputs(scaled(WORKLOADS["base_coherent"], B=2, Q=Q), seed=Q)
    got = _gpu_one_stage(inp, dev)
    want = _oracle_one_stage(oracle, inp)
    for i in (0, 1, 4, 5):
        torch.testing.assert_close(got[i], want[i], **(F32_FWD if i < 2 else F32_BWD))
    _assert_sums_within_term_count_bound(oracle, inp, got[2], got[3])
    got2 = _gpu_two_stage(inp, dev, sliced=False)
    for i in (0, 1, 4, 5):
        torch.testing.assert_close(got2[i], want[i], **(F32_FWD if i < 2 else F32_BWD))
    _assert_sums_within_term_count_bound(oracle, inp, got2[2], got2[3])


class _OptionsSeen:
    """Records the launch options every library call made inside the block actually carries (on whatever thread
    the call is made: the backward of a Function runs on the autograd engine's thread)."""

    def __enter__(self):
        from dfa3D import _lib
        self._lib, self._orig, self.calls = _lib, _lib.options, []

        def recording():
            self.calls.append(self._lib.current_fields())
            return self._orig()
        _lib.options = recording
        return self

    def __exit__(self, *exc):
        self._lib.options = self._orig

    def assert_all_carry(self, setting, at_least):
        want = {("pass_" if k == "pass" else k): v for k, v in setting.items()}
        assert len(self.calls) >= at_least, f"{len(self.calls)} library calls seen, expected at least {at_least}"
        for c in self.calls:
            assert all(c.get(k) == v for k, v in want.items()), f"a library call carried {c}, not {want}"


def _gpu_two_stage(inp, dev, sliced):
    """The reference's two-stage composition; `sliced` hands the 2-D stage (L,2) shapes and (…,2)
    locations as the reference does, otherwise the 3-wide tensors go in as they are."""
    _, F3, F2 = _functions()
    value = inp["value"].to(dev).requires_grad_()
    dist = inp["value_dpt_dist"].to(dev).requires_grad_()
    loc3 = inp["sampling_locations"].to(dev).requires_grad_()
    attn = inp["attention_weights"].to(dev).requires_grad_()
    shapes3, lsi = inp["spatial_shapes"].to(dev), inp["level_start_index"].to(dev)
    score = F3.apply(dist, shapes3, lsi, loc3, 64)
    if sliced:
        out = F2.apply(value, shapes3[:, :2].contiguous(), lsi, loc3[..., :2].contiguous(), attn, score, 64)
    else:
        out = F2.apply(value, shapes3, lsi, loc3, attn, score, 64)
    gv, gd, gl, ga = torch.autograd.grad(out, [value, dist, loc3, attn], inp["grad_output"].to(dev))
    torch.cuda.synchronize()
    return out.detach().cpu(), score.detach().cpu(), gv.cpu(), gd.cpu(), gl.cpu(), ga.cpu()


@pytest.mark.parametrize("binned", [1, 0], ids=["tiles", "atomics"])
@pytest.mark.parametrize("sliced", [True, False], ids=["sliced", "wide"])
def test_fp32_two_stage_workloads_match_checker(oracle, binned, sliced):
    """Both backward implementations of the two separate stages (LDS tiles with a workspace, and
    device-memory atomics), with 2-wide and 3-wide shape / location operands."""
    from dfa3D import _lib
    from dfa3D.workloads import WORKLOADS, make_inputs
    dev = _dev()
    setting = dict(direct=0 if binned else 1)
    with _lib.launch_options(**setting), _OptionsSeen() as seen:
        for name in ("unit", "small"):
            inp = make_inputs(WORKLOADS[name])
            _compare(_gpu_two_stage(inp, dev, sliced), _oracle_one_stage(oracle, inp), F32_FWD, F32_BWD)
    seen.assert_all_carry(setting, at_least=8)         # two forwards and two backwards per workload
    # and the option decides the path: no workspace is asked for when the device-atomics kernels are wanted
    import ctypes
    o = ctypes.pointer(_lib.LaunchOptions(**setting))
    ws = _lib.lib().dfa3d_wms_deform_attn_backward_workspace_bytes(6, 920, 8, 32, 1, 4000, 8, _lib.DFA3D_F32, o)
    assert (ws > 0) == bool(binned)


@pytest.mark.parametrize("seed", [500, 504, 508, 509])
def test_fp32_medium_shapes_clustered_locations(oracle, seed):
    """0.16 M to 5.2 M points on maps of many tiles, locations drawn around the map centre (sigma 0.04): a few
    bins hold most points and are split over several work items; 12 heads put two heads on one queue."""
    import random
    dev = _dev()
    r = random.Random(seed)
    L = r.randint(1, 4)
    levels = tuple((r.randint(8, 120), r.randint(8, 200)) for _ in range(L))
    case = dict(seed=seed, B=r.randint(1, 3), M=r.choice([3, 8, 12]), C=r.choice([16, 32, 64]), D=r.choice([16, 64, 128]),
                Q=r.randint(500, 5000), P=r.choice([4, 8]), levels=levels, dtype=torch.float32)
    print("case", case, flush=True)
    t = tiny_case(**case)
    g = torch.Generator().manual_seed(seed)
    t["loc"] = (0.5 + 0.04 * torch.randn(t["loc"].shape, generator=g)).contiguous()
    inp = _as_inputs(t)
    got = _gpu_one_stage(inp, dev)
    want = _oracle_one_stage(oracle, inp)
    for i in (0, 1, 4, 5):                                   # output, depth_score, grad_loc, grad_attn
        torch.testing.assert_close(got[i], want[i], **(F32_FWD if i < 2 else F32_BWD))
    # thousands of terms per grad_value / grad_dist element: held against the float64 checker
    _assert_sums_within_term_count_bound(oracle, inp, got[2], got[3])


@pytest.mark.parametrize("seed", range(130, 142))
def test_fp32_random_shapes_two_stage_and_shared_distribution(oracle, seed):
    """The drawn shapes of _random_case through the two separate stages (3-wide and sliced operands) and
    through the shared-distribution Function with a gradient at weight_update."""
    from dfa3D.functional import MultiScale3DDeformableAttnWeightUpdateFunction
    dev = _dev()
    case = _random_case(seed)
    print("case", case, flush=True)
    t = tiny_case(**case)
    inp = {k: (v.float() if v.is_floating_point() else v) for k, v in _as_inputs(t).items()}
    want = _oracle_one_stage(oracle, inp)
    _compare(_gpu_two_stage(inp, dev, sliced=seed % 2 == 0), want, F32_FWD, F32_BWD)

    shared = dict(inp)
    shared["value_dpt_dist"] = inp["value_dpt_dist"][:, :, :1].contiguous()
    g = torch.Generator().manual_seed(seed)
    grad_wu = torch.randn(*inp["attention_weights"].shape[:3], 1, generator=g)
    want = _shared_dist_expectation(oracle, shared, grad_wu=grad_wu)
    v, d, loc, a = [shared[k].to(dev).requires_grad_() for k in ("value", "value_dpt_dist", "sampling_locations",
                                                                  "attention_weights")]
    out, wu = MultiScale3DDeformableAttnWeightUpdateFunction.apply(
        v, d, shared["spatial_shapes"].to(dev), shared["level_start_index"].to(dev), loc, a, 64)
    grads = torch.autograd.grad([out, wu], [v, d, loc, a], [shared["grad_output"].to(dev), grad_wu.to(dev)])
    torch.testing.assert_close(wu.detach().cpu(), want[2], **F32_FWD)
    _compare([out.detach().cpu(), want[1], *[x.cpu() for x in grads]], [want[0], want[1], *want[3:]], F32_FWD, F32_BWD)


@pytest.mark.parametrize("setting", [dict(block=256), dict(**{"pass": 128}), dict(**{"pass": 64}), dict(tile=404),
                                     dict(tile=816), dict(tile=203, chunk=64), dict(chunk=256), dict(vec=4),
                                     dict(vec=8, tile=404), dict(iters=3), dict(tile=608), dict(tile=408, chunk=100),
                                     dict(tile=202), dict(tile=101, chunk=64)],
                         ids=lambda d: "-".join(f"{k}{v}" for k, v in d.items()))
def test_launch_options_do_not_change_results(oracle, setting):
    """Tile shape, workgroup size, points per pass, points per work item and channels per lane of the binned
    backward are launch parameters only."""
    from dfa3D import _lib
    dev = _dev()
    t = tiny_case(70, B=2, C=32, M=8, Q=700, P=8, D=16, levels=((37, 52), (19, 26), (7, 9)), dtype=torch.float32)
    inp = _as_inputs(t)
    want = _oracle_one_stage(oracle, inp)
    with _lib.launch_options(**setting), _OptionsSeen() as seen:
        _compare(_gpu_one_stage(inp, dev), want, F32_FWD, F32_BWD)
        _compare(_gpu_two_stage(inp, dev, sliced=False), want, F32_FWD, F32_BWD)
    seen.assert_all_carry(setting, at_least=6)         # one forward + one backward, then two of each


@pytest.mark.parametrize("variant", ["tiles", "many-items", "odd-channels", "direct", "fp64", "shared", "bf16", "gap",
                                     "static"])
def test_gradient_buffers_that_were_not_zeroed(variant):
    """options.clear: grad_value / grad_dist handed over full of NaN come back equal to what the call writes into
    zeroed buffers, on the tile kernels (one work item per tile, several, tiles without points, rows that are
    no whole 16-byte groups, keys that belong to no level), on the direct kernels, for a distribution shared by the
    heads, for bfloat16 gradient buffers and through the entry point with the built-in scratch."""
    import ctypes
    from dfa3D import _ext, _lib
    dev = _dev()
    kw = dict(seed=300, B=2, M=8, C=32, D=16, Q=400, P=4, levels=((37, 52), (19, 26), (5, 3)), dtype=torch.float32)
    opts = {}
    if variant == "many-items":
        opts = dict(chunk=64)
    elif variant == "odd-channels":
        kw.update(C=6, D=5)
    elif variant == "direct":
        opts = dict(direct=1)
    elif variant == "fp64":
        kw.update(dtype=torch.float64, Q=60)
    t = tiny_case(**kw)
    t["loc"][:, :, :, 0] = t["loc"][:, :, :, 0] * 0.3            # level 0: most tiles stay without points
    value, dist, loc, attn, go = [t[k].to(dev) for k in ("value", "dist", "loc", "attn", "grad_out")]
    shapes3, lsi = t["shapes3"].to(dev), t["lsi"].to(dev)
    if variant == "gap":                                         # seven keys between the levels belong to no level
        cut = int(lsi[1])
        pad = lambda x: torch.cat([x[:, :cut], torch.randn_like(x[:, :7]), x[:, cut:]], 1).contiguous()
        value, dist = pad(value), pad(dist)
        lsi = lsi.clone()
        lsi[1:] += 7
    if variant == "shared":
        dist = dist[:, :, :1].contiguous()
    gdt = value.dtype
    if variant == "bf16":
        value, dist, go = value.bfloat16(), dist.bfloat16(), go.bfloat16()
        gdt = _ext.fused_backward_grad_dtype(value, dist, loc)
        assert gdt == torch.bfloat16

    def run(fill, clear):
        gv = torch.full(value.shape, fill, dtype=gdt, device=dev)
        gd = torch.full(dist.shape, fill, dtype=gdt, device=dev)
        gl, ga = torch.empty_like(loc), torch.empty_like(attn)
        with _lib.launch_options(**opts):
            if variant == "static":
                B, S, M, C = value.shape
                o = ctypes.pointer(_lib.LaunchOptions(clear=1 if clear else 0))
                rc = _lib.lib().dfa3d_fused_backward_static(
                    _lib.ptr(value), _lib.ptr(dist), _lib.ptr(shapes3), _lib.ptr(lsi), _lib.ptr(loc), _lib.ptr(attn),
                    _lib.ptr(go), None, None, _lib.ptr(gv), _lib.ptr(gd), _lib.ptr(gl), _lib.ptr(ga), B, S, M, C,
                    dist.shape[3], loc.shape[3], loc.shape[1], loc.shape[4], dist.shape[2], _lib.dtype_code(value), o,
                    _lib.stream_of(value))
                _lib.check(rc, "dfa3d_fused_backward_static")
            else:
                _ext.dfa3d_fused_backward(value, dist, shapes3, lsi, loc, attn, go, None, gv, gd, gl, ga, 64, clear=clear)
        torch.cuda.synchronize()
        return gv.float().cpu(), gd.float().cpu()

    want_gv, want_gd = run(0.0, False)
    got_gv, got_gd = run(float("nan"), True)
    assert torch.isfinite(got_gv).all() and torch.isfinite(got_gd).all()
    tol = dict(rtol=2e-2, atol=2e-2) if variant == "bf16" else dict(rtol=1e-5, atol=1e-5)    # order of the atomic adds
    torch.testing.assert_close(got_gv, want_gv, **tol)
    torch.testing.assert_close(got_gd, want_gd, **tol)
    assert want_gv.abs().sum() > 0 and want_gd.abs().sum() > 0


@pytest.mark.parametrize("variant", ["scores", "plain", "plain-direct", "odd-channels"])
def test_stage_two_gradient_buffer_that_was_not_zeroed(variant):
    """options.clear on the stage-2 backward (depth scores given, or none: plain deformable attention): a grad_value
    full of NaN comes back equal to what the call writes into a zeroed one."""
    from dfa3D import _ext, _lib
    dev = _dev()
    kw = dict(seed=310, B=2, M=8, C=32, D=4, Q=400, P=4, levels=((37, 52), (19, 26), (5, 3)), dtype=torch.float32)
    if variant == "odd-channels":
        kw.update(C=6)
    t = tiny_case(**kw)
    t["loc"][:, :, :, 0] = t["loc"][:, :, :, 0] * 0.3            # level 0: most tiles stay without points
    value, loc, attn, go = [t[k].to(dev) for k in ("value", "loc", "attn", "grad_out")]
    shapes3, lsi = t["shapes3"].to(dev), t["lsi"].to(dev)
    score = torch.rand(*attn.shape, 4, device=dev)
    opts = dict(direct=1) if variant == "plain-direct" else {}

    def run(fill, clear):
        gv = torch.full(value.shape, fill, device=dev)
        gl, ga, gs = torch.zeros_like(loc), torch.empty_like(attn), torch.empty_like(score)
        with _lib.launch_options(**opts):
            if variant.startswith("plain"):
                _ext.ms_deform_attn_backward(value, shapes3, lsi, loc, attn, go, gv, gl, ga, 64, clear=clear)
            else:
                _ext.wms_deform_attn_backward_into(value, shapes3, lsi, loc, attn, score, go, gv, gl, ga, gs, 64, clear=clear)
        torch.cuda.synchronize()
        return gv.cpu()

    want, got = run(0.0, False), run(float("nan"), True)
    assert torch.isfinite(got).all() and want.abs().sum() > 0
    torch.testing.assert_close(got, want, rtol=1e-5, atol=1e-5)


def _random_case_with_options(seed):
    """A wider draw than _random_case (channel counts up to 256, depth bins up to 128, up to 3000 queries on maps of
    1 to 60 pixels a side, locations inside, around and in a corner of the map) with launch options drawn from
    what the library accepts."""
    import random
    r = random.Random(seed)
    L = r.randint(1, 5)
    side = 60 if r.random() < 0.4 else 24
    levels = tuple((r.randint(1, side), r.randint(1, side)) for _ in range(L))
    case = dict(seed=seed, B=r.randint(1, 3), M=r.choice([1, 2, 3, 4, 5, 7, 8, 9, 16]),
                C=r.choice([1, 2, 3, 4, 8, 12, 16, 20, 24, 32, 36, 40, 48, 64, 72, 96, 128, 160, 256]),
                D=r.choice([1, 2, 3, 4, 7, 8, 16, 17, 32, 48, 64, 80, 112, 128]),
                Q=r.choice([1, 2, 7, 33, 100, 257, 600, 1500, 3000]), P=r.randint(1, 9), levels=levels,
                lo=r.choice([0.0, -0.2, 0.3]), hi=r.choice([1.0, 1.2, 0.6]))
    points = case["B"] * case["Q"] * case["M"] * L * case["P"]
    if points * case["C"] > 3e8 or points > 3e6:
        case["Q"] = max(1, case["Q"] // 10)
    opts = {}
    if r.random() < 0.6:
        for name, p, choices in (("tile", 0.5, [202, 203, 404, 408, 804, 808, 816, 1616, 302, 505]),
                                 ("block", 0.3, [256, 512]), ("pass_", 0.3, [64, 128, 256]),
                                 ("chunk", 0.3, [64, 100, 256, 1000, 4096]), ("vec", 0.3, [1, 2, 4, 8]),
                                 ("iters", 0.2, [1, 2, 3, 5]), ("direct", 0.1, [1])):
            if r.random() < p:
                opts[name] = r.choice(choices)
    return case, opts


@pytest.mark.parametrize("seed", range(7000, 7048))
def test_fp32_random_shapes_with_random_launch_options(oracle, seed):
    """One-stage and two-stage paths on drawn shapes under drawn launch options.  Every tensor within the bound that
    follows from the number of terms of its sums, against the float64 checker (dot products over up to 256 channels
    scaled by the map size are outside the flat 1e-5 / 1e-4 gates of the headline shapes, and inside this one)."""
    from dfa3D import _lib
    dev = _dev()
    case, opts = _random_case_with_options(seed)
    print("case", case, "options", opts, flush=True)
    t = tiny_case(**case)
    inp = {k: (v.float() if v.is_floating_point() else v) for k, v in _as_inputs(t).items()}
    with _lib.launch_options(**opts):
        results = (_gpu_one_stage(inp, dev), _gpu_two_stage(inp, dev, sliced=seed % 2 == 0))
    for got in results:
        _assert_per_point_within_term_count_bound(oracle, inp, got[0], got[1], got[4], got[5])
        _assert_sums_within_term_count_bound(oracle, inp, got[2], got[3])


def test_fp32_base_shape_two_stage_matches_checker(oracle):
    from dfa3D.workloads import WORKLOADS, make_inputs
    dev = _dev()
    inp = make_inputs(WORKLOADS["base"])
    _compare(_gpu_two_stage(inp, dev, sliced=False), _oracle_one_stage(oracle, inp), F32_FWD, F32_BWD)


def test_fp32_base_shape_matches_checker(oracle):
    """BEVFormer-base shape at full size (15.36 M sampling points)."""
    from dfa3D.workloads import WORKLOADS, make_inputs
    dev = _dev()
    inp = make_inputs(WORKLOADS["base"])
    got = _gpu_one_stage(inp, dev)
    want = _oracle_one_stage(oracle, inp)
    _compare(got, want, F32_FWD, F32_BWD)


def _inner(a, b):
    return (a.double() * b.double()).sum().item()


def test_fp32_dense_shape_properties():
    """Dense BEV stress shape (61.44 M points): size-independent identities (the comparison with the checker is
    test_dense_shape_full_size_matches_checker).  The operator is linear in value, in the depth distributions and
    in the attention weights, so <x, dL/dx> = <output, grad_output> for each of them (Euler), and
    the two-stage chain must reproduce the one-stage result."""
    from dfa3D.workloads import WORKLOADS, make_inputs
    dev = _dev()
    F1, F3, F2 = _functions()
    inp = make_inputs(WORKLOADS["dense"], device=dev)
    value = inp["value"].requires_grad_()
    dist = inp["value_dpt_dist"].requires_grad_()
    loc = inp["sampling_locations"]
    attn = inp["attention_weights"].requires_grad_()
    shapes3, lsi = inp["spatial_shapes"], inp["level_start_index"]
    out, score = F1.apply(value, dist, shapes3, lsi, loc, attn, 64)
    go = inp["grad_output"]
    gv, gd, ga = torch.autograd.grad(out, [value, dist, attn], go)
    ref = _inner(out, go)
    scale = (out.double().abs() * go.double().abs()).sum().item()
    for name, x, gx in (("value", value, gv), ("dist", dist, gd), ("attn", attn, ga)):
        assert abs(_inner(x, gx) - ref) <= 1e-5 * scale, name
    with torch.no_grad():
        score2 = F3.apply(dist.detach(), shapes3, lsi, loc, 64)
        assert torch.equal(score2, score)
        out2 = F2.apply(value.detach(), shapes3[:, :2].contiguous(), lsi, loc[..., :2].contiguous(),
                        attn.detach(), score2, 64)
        torch.testing.assert_close(out2, out.detach(), **F32_FWD)
        # linearity in value at full size
        out3, _ = F1.apply(value.detach() * 2 + 1, dist.detach(), shapes3, lsi, loc, attn.detach(), 64)
        ones, _ = F1.apply(torch.ones_like(value), dist.detach(), shapes3, lsi, loc, attn.detach(), 64)
        torch.testing.assert_close(out3, 2 * out.detach() + ones, rtol=1e-4, atol=1e-5)


def _bf16_one_stage_check(oracle, inp, dev):
    """bfloat16 value / distributions / grad_output, float32 locations and weights, float32 accumulation, against
    the checker run on the bf16-ROUNDED inputs.  The only extra error is the bf16 rounding of what is stored in
    bf16: output and depth_score (2^-8 relative, stated bound rtol = atol = 8e-3 against the float32 checker),
    and the returned value / dist gradients (float32 sums in LDS, rounded to bf16 as the tiles are written: the
    term-count bound of the float32 tests plus 2^-8 relative, plus the packed bf16 atomics on shared rows).
    grad_loc and grad_attn stay float32 and keep the float32 tolerance."""
    F1, _, _ = _functions()
    v16, d16 = inp["value"].bfloat16(), inp["value_dpt_dist"].bfloat16()
    go16 = inp["grad_output"].bfloat16()
    value, dist = v16.to(dev).requires_grad_(), d16.to(dev).requires_grad_()
    loc, attn = inp["sampling_locations"].to(dev).requires_grad_(), inp["attention_weights"].to(dev).requires_grad_()
    out, score = F1.apply(value, dist, inp["spatial_shapes"].to(dev), inp["level_start_index"].to(dev), loc, attn, 64)
    assert out.dtype == torch.bfloat16 and score.dtype == torch.bfloat16
    gv, gd, gl, ga = torch.autograd.grad(out, [value, dist, loc, attn], go16.to(dev))
    assert gv.dtype == torch.bfloat16 and gd.dtype == torch.bfloat16 and gl.dtype == torch.float32
    ref = dict(inp, value=v16.float(), value_dpt_dist=d16.float(), grad_output=go16.float())
    o_out, o_score, o_gv, o_gd, o_gl, o_ga = _oracle_one_stage(oracle, ref)
    bf = dict(rtol=8e-3, atol=8e-3)
    torch.testing.assert_close(out.float().cpu(), o_out, **bf)
    torch.testing.assert_close(score.float().cpu(), o_score, **bf)
    torch.testing.assert_close(gl.cpu(), o_gl, **F32_BWD)
    torch.testing.assert_close(ga.cpu(), o_ga, **F32_BWD)
    # bins of up to 3 work items (4096 points each) on rows shared by up to 4 tiles: 12 rounding adds at most
    _assert_sums_within_term_count_bound(oracle, ref, gv.float().cpu(), gd.float().cpu(), storage_rel=2.0 ** -8,
                                         atomic_rel=12 * 2.0 ** -9)


def test_bf16_storage(oracle):
    """Reduced size (B=2, Q=1500) of the peaky-depth workload."""
    from dfa3D.workloads import WORKLOADS, make_inputs, scaled
    _bf16_one_stage_check(oracle, make_inputs(scaled(WORKLOADS["base_peaky"], B=2, Q=1500), seed=4), _dev())


def test_bf16_storage_full_base_shape(oracle):
    """The whole bf16 configuration: BEVFormer-base shape (B=6, Q=10000, 15.36 M points), peaky depth."""
    from dfa3D.workloads import WORKLOADS, make_inputs
    _bf16_one_stage_check(oracle, make_inputs(WORKLOADS["base_peaky"]), _dev())


@pytest.mark.parametrize("case", [dict(seed=60, C=6, M=3, Q=17, P=3, D=5, levels=((7, 5), (3, 4))),
                                  dict(seed=61, C=16, M=2, Q=9, P=5, D=7, levels=((4, 9),)),
                                  dict(seed=62, C=1, M=2, Q=5, P=2, D=2, levels=((3, 3), (2, 2)))],
                         ids=lambda c: f"seed{c['seed']}")
def test_bf16_odd_shapes(oracle, case):
    """bfloat16 storage with row lengths that rule out the aligned vector loads (odd D, C = 1 / 6 / 16)."""
    dev = _dev()
    F1, _, _ = _functions()
    t = tiny_case(dtype=torch.float32, **case)
    inp = _as_inputs(t)
    r16 = dict(inp, value=inp["value"].bfloat16().float(), value_dpt_dist=inp["value_dpt_dist"].bfloat16().float(),
               grad_output=inp["grad_output"].bfloat16().float())
    value = inp["value"].bfloat16().to(dev).requires_grad_()
    dist = inp["value_dpt_dist"].bfloat16().to(dev).requires_grad_()
    loc, attn = inp["sampling_locations"].to(dev).requires_grad_(), inp["attention_weights"].to(dev).requires_grad_()
    out, score = F1.apply(value, dist, inp["spatial_shapes"].to(dev), inp["level_start_index"].to(dev), loc, attn, 64)
    gv, gd, gl, ga = torch.autograd.grad(out, [value, dist, loc, attn], inp["grad_output"].bfloat16().to(dev))
    o_out, o_score, o_gv, o_gd, o_gl, o_ga = _oracle_one_stage(oracle, r16)
    bf = dict(rtol=8e-3, atol=8e-3)
    torch.testing.assert_close(out.float().cpu(), o_out, **bf)
    torch.testing.assert_close(score.float().cpu(), o_score, **bf)
    torch.testing.assert_close(gl.cpu(), o_gl, **F32_BWD)
    torch.testing.assert_close(ga.cpu(), o_ga, **F32_BWD)
    _assert_sums_within_term_count_bound(oracle, r16, gv.float().cpu(), gd.float().cpu(), storage_rel=2.0 ** -8,
                                         atomic_rel=4 * 2.0 ** -9)


def test_bf16_other_entry_points(oracle):
    """bfloat16 storage through the two separate stages, through the shared-distribution / weight_update
    Function and through plain deformable attention, same bounds as test_bf16_storage."""
    from dfa3D.functional import MultiScale3DDeformableAttnWeightUpdateFunction, MultiScaleDeformableAttnFunction
    from dfa3D.workloads import WORKLOADS, make_inputs, scaled
    dev = _dev()
    w = scaled(WORKLOADS["base_peaky"], B=2, Q=700)
    inp = make_inputs(w, seed=6)
    bf = dict(rtol=8e-3, atol=8e-3)
    r16 = dict(inp, value=inp["value"].bfloat16().float(), value_dpt_dist=inp["value_dpt_dist"].bfloat16().float(),
               grad_output=inp["grad_output"].bfloat16().float())
    shapes3, lsi = inp["spatial_shapes"].to(dev), inp["level_start_index"].to(dev)

    def leaves(dist):
        return [inp["value"].bfloat16().to(dev).requires_grad_(), dist.bfloat16().to(dev).requires_grad_(),
                inp["sampling_locations"].to(dev).requires_grad_(), inp["attention_weights"].to(dev).requires_grad_()]


    # two stages, score tensor stored in bf16 between them
    _, F3, F2 = _functions()
    o_out, o_score, o_gv, o_gd, o_gl, o_ga = _oracle_one_stage(oracle, r16)
    v, d, loc, a = leaves(inp["value_dpt_dist"])
    score = F3.apply(d, shapes3, lsi, loc, 64)
    out = F2.apply(v, shapes3, lsi, loc, a, score, 64)
    assert score.dtype == torch.bfloat16 and out.dtype == torch.bfloat16
    grads = torch.autograd.grad(out, [v, d, loc, a], inp["grad_output"].bfloat16().to(dev))
    # Every term of the output and of the per-point gradients carries the rounding of the score tensor stored in
    # bfloat16 between the two kernels (2^-8 relative), the z gradient also that of the scores' gradient on the way
    # back (another 2^-8); output and scores are themselves stored in bfloat16.  grad_loc / grad_attn are float32.
    _assert_per_point_within_term_count_bound(oracle, r16, out.float().cpu(), score.float().cpu(), grads[2].cpu(),
                                              grads[3].cpu(), term_rel=2.0 ** -7, storage_rel=2.0 ** -8)
    # every term of both sums carries the rounding of a tensor stored in bf16 between the two kernels (the scores
    # on the way forward, their gradient on the way back): 2^-8 relative each
    _assert_sums_within_term_count_bound(oracle, r16, grads[0].float().cpu(), grads[1].float().cpu(),
                                         storage_rel=2.0 ** -8, term_rel=2.0 ** -7)

    # one distribution for all heads, weight_update instead of scores
    shared = dict(r16, value_dpt_dist=r16["value_dpt_dist"][:, :, :1].contiguous())
    want = _shared_dist_expectation(oracle, shared)
    v, d, loc, a = leaves(inp["value_dpt_dist"][:, :, :1].contiguous())
    out, wu = MultiScale3DDeformableAttnWeightUpdateFunction.apply(v, d, shapes3, lsi, loc, a, 64)
    grads = torch.autograd.grad(out, [v, d, loc, a], inp["grad_output"].bfloat16().to(dev))
    torch.testing.assert_close(out.float().cpu(), want[0], **bf)
    torch.testing.assert_close(wu.cpu(), want[2], **F32_FWD)
    torch.testing.assert_close(grads[2].cpu(), want[5], **F32_BWD)
    torch.testing.assert_close(grads[3].cpu(), want[6], **F32_BWD)
    rep16 = dict(r16, value_dpt_dist=shared["value_dpt_dist"].repeat(1, 1, inp["value"].shape[2], 1).contiguous())
    _assert_sums_within_term_count_bound(oracle, rep16, grads[0].float().cpu(), grads[1].float().cpu(),
                                         storage_rel=2.0 ** -8, shared_dist=True, atomic_rel=4 * 2.0 ** -9)

    # plain deformable attention
    ones = torch.ones(*inp["attention_weights"].shape, 4)
    args = (r16["value"], inp["spatial_shapes"][:, :2].contiguous(), inp["level_start_index"],
            inp["sampling_locations"][..., :2].contiguous(), inp["attention_weights"], ones)
    p_out = oracle.wms_forward(*args)
    p_gv, p_gl, p_ga, _ = oracle.wms_backward(*args, r16["grad_output"])
    v, _, loc, a = leaves(inp["value_dpt_dist"])
    out = MultiScaleDeformableAttnFunction.apply(v, shapes3, lsi, loc, a, 64)
    gv, gl, ga = torch.autograd.grad(out, [v, loc, a], inp["grad_output"].bfloat16().to(dev))
    torch.testing.assert_close(out.float().cpu(), p_out, **bf)
    torch.testing.assert_close(gv.float().cpu(), p_gv, **bf)
    torch.testing.assert_close(gl[..., :2].cpu(), p_gl, **F32_BWD)
    torch.testing.assert_close(ga.cpu(), p_ga, **F32_BWD)


@pytest.mark.parametrize("dtype", [torch.float64, torch.float32], ids=["fp64", "fp32"])
def test_degenerate_level_shapes_and_sixteen_levels(oracle, dtype):
    """Levels of one pixel, one row, one column; the maximum of 16 levels."""
    dev = _dev()
    tol = (dict(rtol=1e-10, atol=1e-11),) * 2 if dtype == torch.float64 else (F32_FWD, F32_BWD)
    shapes = [((1, 1), (1, 5), (7, 1), (2, 2)),
              tuple((1 + i % 3, 1 + (i * 5) % 4) for i in range(16))]
    for i, levels in enumerate(shapes):
        t = tiny_case(40 + i, C=8, M=2, Q=13, P=2, D=4, levels=levels, dtype=dtype)
        inp = _as_inputs(t)
        _compare(_gpu_one_stage(inp, dev), _oracle_one_stage(oracle, inp), *tol)


def test_nothing_sampled_and_nothing_asked(oracle):
    """Every location outside every map: zeros everywhere.  No queries at all: empty results, zero gradients."""
    dev = _dev()
    F1, _, _ = _functions()
    t = tiny_case(50, C=32, M=2, Q=9, P=4, levels=((6, 7), (3, 3)), dtype=torch.float32, lo=1.5, hi=2.5)
    got = _gpu_one_stage(_as_inputs(t), dev)
    for g in got:
        assert g.abs().max().item() == 0
    value = t["value"].to(dev).requires_grad_()
    dist = t["dist"].to(dev).requires_grad_()
    loc = t["loc"][:, :0].contiguous().to(dev).requires_grad_()
    attn = t["attn"][:, :0].contiguous().to(dev).requires_grad_()
    out, score = F1.apply(value, dist, t["shapes3"].to(dev), t["lsi"].to(dev), loc, attn, 64)
    assert out.shape == (2, 0, 64) and score.shape == (2, 0, 2, 2, 4, 4)
    gv, gd, gl, ga = torch.autograd.grad(out, [value, dist, loc, attn], torch.zeros_like(out))
    assert gv.abs().max().item() == 0 and gd.abs().max().item() == 0 and gl.numel() == 0 and ga.numel() == 0


def test_more_tiles_than_the_block_histogram_holds(oracle):
    """A 760 x 700 map has 8360 tiles per (batch, head): more than the binning blocks count in LDS, so they
    count in device memory."""
    dev = _dev()
    t = tiny_case(56, B=1, C=4, M=2, Q=3000, P=4, D=2, levels=((760, 700), (3, 5)), dtype=torch.float32)
    inp = _as_inputs(t)
    _compare(_gpu_one_stage(inp, dev), _oracle_one_stage(oracle, inp), F32_FWD, F32_BWD)


@pytest.mark.parametrize("case", [dict(seed=57, B=1, C=4, M=2, Q=2000, P=4, D=2, levels=((400, 410), (3, 5))),
                                  dict(seed=58, B=2, C=8, M=3, Q=5, P=2100, D=4, levels=((30, 41),)),
                                  dict(seed=59, B=1, C=8, M=9, Q=3, P=700, D=3, levels=((9, 9), (20, 17), (5, 4)))],
                         ids=["2600-tiles", "2100-points-per-unit", "2100-points-per-unit-3-levels"])
def test_binning_fallbacks(oracle, case):
    """Shapes the block-sorted binning kernels leave to the plain ones: more than 2048 tiles per (batch, head)
    (counted in LDS by the plain kernels up to 8192 tiles), and more than 2048 sampling points per unit."""
    dev = _dev()
    t = tiny_case(dtype=torch.float32, **case)
    inp = _as_inputs(t)
    _compare(_gpu_one_stage(inp, dev), _oracle_one_stage(oracle, inp), F32_FWD, F32_BWD)


def test_every_point_in_one_pixel_cell(oracle):
    """All sampling points in the same pixel cell and depth interval: one tile gets everything (several work
    items for one bin, every tile address contested).  Sums of 12 000 float32 terms, checked against the
    float64 checker with the bound that follows from the number of terms."""
    dev = _dev()
    t = tiny_case(55, B=1, C=32, M=2, Q=1500, P=4, D=16, levels=((20, 30),), dtype=torch.float32)
    g = torch.Generator().manual_seed(5)
    loc = torch.tensor([0.37, 0.52, 0.41]) + (torch.rand(t["loc"].shape, generator=g) - 0.5) * 0.01
    inp = dict(_as_inputs(t), sampling_locations=loc.contiguous())
    got = _gpu_one_stage(inp, dev)
    want = _oracle_one_stage(oracle, inp)
    for i in (0, 1, 4, 5):
        torch.testing.assert_close(got[i], want[i], **(F32_FWD if i < 2 else F32_BWD))
    _assert_sums_within_term_count_bound(oracle, inp, got[2], got[3])


def test_non_finite_and_huge_locations_are_skipped(oracle):
    """NaN, infinite and absurdly large coordinates fail the reference's range tests (every comparison with a
    NaN is false, cuh:69 / cuh:262) and contribute nothing; no index derived from them is ever used."""
    dev = _dev()
    t = tiny_case(31, C=32, M=2, Q=40, P=4, levels=((9, 11), (5, 6)), dtype=torch.float32)
    loc = t["loc"].clone()
    flat = loc.view(-1, 3)
    bad = [float("nan"), float("inf"), float("-inf"), 1e30, -1e30, 3e9, -3e9]
    for i, v in enumerate(bad * 3):
        flat[7 * i + 3, i % 3] = v
    inp = dict(_as_inputs(t), sampling_locations=loc)
    got = _gpu_one_stage(inp, dev)
    want = _oracle_one_stage(oracle, inp)
    for g in got:
        assert torch.isfinite(g).all()
    _compare(got, want, F32_FWD, F32_BWD)


def test_nan_in_unsampled_pixel_does_not_leak(oracle):
    """Corners outside the map are never read and never multiplied in."""
    dev = _dev()
    t = tiny_case(20, C=32, M=1, Q=3, P=2, levels=((4, 4),), lo=0.3, hi=0.7)
    inp = _as_inputs(t)
    inp["value"][:, 0] = float("nan")          # pixel (0, 0): no location in [0.3, 0.7]^2 touches it
    inp["sampling_locations"][0, 0, 0, 0, 0, :2] = torch.tensor([1.1, 0.5], dtype=torch.float64)   # RT/RB outside
    got = _gpu_one_stage(inp, dev)
    want = _oracle_one_stage(oracle, inp)
    assert torch.isfinite(got[0]).all()
    torch.testing.assert_close(got[0], want[0], rtol=1e-10, atol=1e-11)


def test_inconsistent_level_table_is_contained():
    """A level that does not fit in the key dimension is treated as empty instead of reading out of
    bounds (the reference would read past the tensor)."""
    dev = _dev()
    F1, _, _ = _functions()
    t = tiny_case(21, C=32, M=2, Q=4, P=2, levels=((4, 4), (2, 2)))
    bad = t["shapes3"].clone()
    bad[1, 0] = 50                       # 50 x 2 keys do not fit
    out, score = F1.apply(t["value"].to(dev), t["dist"].to(dev), bad.to(dev), t["lsi"].to(dev),
                          t["loc"].to(dev), t["attn"].to(dev), 64)
    torch.cuda.synchronize()
    assert torch.isfinite(out).all() and score[:, :, :, 1].abs().max().item() == 0


def test_non_finite_grad_output_stays_in_the_rows_it_touches(oracle):
    """One infinite element in grad_output: the reference's backward makes non-finite exactly the grad_value rows
    and grad_dist bins that the unit's own sampling points touch.  Everything else must stay finite and right:
    lanes of the tile kernel that idle while their wavefront finishes a longer task list must not multiply
    another point's staged gradient (0 * inf) into their row."""
    dev = _dev()
    t = tiny_case(81, B=1, C=32, M=2, Q=600, P=4, D=8, levels=((24, 31), (9, 11)), dtype=torch.float32, lo=0.0, hi=1.0)
    inp = _as_inputs(t)
    inp["grad_output"][0, 17, 5] = float("inf")           # unit (b=0, q=17, m=0), channel 5
    got = _gpu_one_stage(inp, dev)
    want = _oracle_one_stage(oracle, inp)
    for name, g, w in (("grad_value", got[2], want[2]), ("grad_dist", got[3], want[3]),
                       ("grad_loc", got[4], want[4]), ("grad_attn", got[5], want[5])):
        clean = torch.isfinite(w)
        assert clean.float().mean().item() > 0.8, name          # the infinity reaches only a few elements
        assert torch.isfinite(g[clean]).all(), f"{name}: non-finite values outside what the unit touches"
        torch.testing.assert_close(g[clean], w[clean], msg=lambda m, n=name: f"{n}: {m}", **F32_BWD)


def test_reference_unittest_operands(oracle):
    """The operands of the reference's own test (unittest_DFA3D.py:43-56: 6 x 30825 keys, 112 depth bins, 9502
    queries, attention weights from U[0,1) that do not sum to one, im2col_step = 32) through the two-stage
    composition and the one-stage Function, as that test calls them (unittest_DFA3D.py:11-28); it only asserts
    "no NaN", here both are compared with the checker and with each other."""
    from dfa3D.workloads import WORKLOADS, make_inputs
    dev = _dev()
    F1, F3, F2 = _functions()
    inp = make_inputs(WORKLOADS["unittest"])
    assert inp["value_dpt_dist"].shape == (6, 30825, 8, 112) and inp["sampling_locations"].shape == (6, 9502, 8, 4, 8, 3)
    want = _oracle_one_stage(oracle, inp)
    value, dist = inp["value"].to(dev).requires_grad_(), inp["value_dpt_dist"].to(dev).requires_grad_()
    loc, attn = inp["sampling_locations"].to(dev).requires_grad_(), inp["attention_weights"].to(dev).requires_grad_()
    shapes3, lsi = inp["spatial_shapes"].to(dev), inp["level_start_index"].to(dev)
    go = inp["grad_output"].to(dev)
    # two stages, sliced operands as in the reference's test
    score = F3.apply(dist, shapes3, lsi, loc, 32)
    out2 = F2.apply(value, shapes3[:, :2].contiguous(), lsi, loc[..., :2].contiguous(), attn, score, 32)
    g2 = torch.autograd.grad(out2, [value, dist, loc, attn], go)
    _compare([out2.detach().cpu(), score.detach().cpu(), *[g.cpu() for g in g2]], want, F32_FWD, F32_BWD)
    # one stage
    out1, score1 = F1.apply(value, dist, shapes3, lsi, loc, attn, 32)
    g1 = torch.autograd.grad(out1, [value, dist, loc, attn], go)
    _compare([out1.detach().cpu(), score1.detach().cpu(), *[g.cpu() for g in g1]], want, F32_FWD, F32_BWD)
    assert torch.equal(score1, score)
    torch.testing.assert_close(out1, out2, **F32_FWD)
    assert not torch.isnan(out1.sum()) and not torch.isnan(out2.sum())          # the reference's own assertion


def test_dense_shape_query_slice_matches_checker(oracle):
    """Dense BEV stress shape at full size (61.44 M points) against the checker on a slice of the queries: units
    are independent in the forward and in the per-point gradients, so output, depth_score, grad_loc and grad_attn
    of the first 500 queries of every batch element must equal what the checker gives for those queries alone."""
    from dfa3D.workloads import WORKLOADS, make_inputs
    dev = _dev()
    F1, _, _ = _functions()
    inp = make_inputs(WORKLOADS["dense"])
    value, dist = inp["value"].to(dev).requires_grad_(), inp["value_dpt_dist"].to(dev).requires_grad_()
    loc, attn = inp["sampling_locations"].to(dev).requires_grad_(), inp["attention_weights"].to(dev).requires_grad_()
    out, score = F1.apply(value, dist, inp["spatial_shapes"].to(dev), inp["level_start_index"].to(dev), loc, attn, 64)
    gl, ga = torch.autograd.grad(out, [loc, attn], inp["grad_output"].to(dev))
    n = 500
    part = dict(inp, sampling_locations=inp["sampling_locations"][:, :n].contiguous(),
                attention_weights=inp["attention_weights"][:, :n].contiguous(),
                grad_output=inp["grad_output"][:, :n].contiguous())
    o_out, o_score, _, _, o_gl, o_ga = _oracle_one_stage(oracle, part)
    torch.testing.assert_close(out[:, :n].detach().cpu(), o_out, **F32_FWD)
    torch.testing.assert_close(score[:, :n].detach().cpu(), o_score, **F32_FWD)
    torch.testing.assert_close(gl[:, :n].cpu(), o_gl, **F32_BWD)
    torch.testing.assert_close(ga[:, :n].cpu(), o_ga, **F32_BWD)


def test_dense_shape_full_size_matches_checker(oracle):
    """The dense BEV stress workload at full size (B=6, Q=40000, 128 depth bins, clustered locations: 61.44 M
    points) against the checker, all six tensors: every bin of the coarse levels takes many passes and several
    work items (tiles flushed with atomic adds, phases of consecutive passes overlapping).  grad_value /
    grad_dist, sums of up to tens of thousands of terms, are held to the term-count bound of the float64 checker."""
    from dfa3D.workloads import WORKLOADS, make_inputs
    dev = _dev()
    inp = make_inputs(WORKLOADS["dense"])
    got = _gpu_one_stage(inp, dev)
    want = _oracle_one_stage(oracle, inp)
    for i in (0, 1, 4, 5):
        torch.testing.assert_close(got[i], want[i], **(F32_FWD if i < 2 else F32_BWD))
    del want
    _assert_sums_within_term_count_bound(oracle, inp, got[2], got[3])


TWINS = ["MultiScale3DDeformableAttnFunction", "WeightedMultiScaleDeformableAttnFunction",
         "MultiScaleDepthScoreSampleFunction"]


@pytest.mark.parametrize("suffix", ["_fp16", "_fp32"])
@pytest.mark.parametrize("base_name", TWINS)
def test_autocast_twins_cast_half_inputs_to_float32(base_name, suffix):
    """The `_fp16` / `_fp32` twins under torch.autocast with float16 operands, as DFA3D-BEVFormer picks them by the
    dtype of `value` (spatial_cross_attention.py:557-564; the reference's twins are
    custom_fwd(cast_inputs=...) wrappers, multi_scale_3ddeformable_attn_function.py:27,106,185,232,278,355):
    floating operands are cast to float32 and the call runs outside autocast, so results equal the base class
    on the float32-cast operands, outputs are float32, and gradients come back in the operands' float16."""
    import dfa3D.functional as fn
    dev = _dev()
    base, twin = getattr(fn, base_name), getattr(fn, base_name + suffix)
    t = tiny_case(91, B=2, C=32, M=8, Q=50, P=8, D=16, levels=((12, 17), (6, 9), (3, 4), (2, 2)), dtype=torch.float32,
                  lo=0.0, hi=1.0)
    half = {k: (v.half() if v.is_floating_point() else v) for k, v in t.items() if torch.is_tensor(v)}
    shapes3, lsi = t["shapes3"].to(dev), t["lsi"].to(dev)
    g = torch.Generator().manual_seed(3)
    score_h = torch.rand(*t["loc"].shape[:-1], 4, generator=g).half()
    gscore = torch.randn(*t["loc"].shape[:-1], 4, generator=g)

    def call(F, cast):
        v, d, loc, a, sc = [cast(x).to(dev).requires_grad_() for x in (half["value"], half["dist"], half["loc"],
                                                                      half["attn"], score_h)]
        if base_name == "MultiScale3DDeformableAttnFunction":
            out, _ = F.apply(v, d, shapes3, lsi, loc, a, 64)
            leaves, gout = [v, d, loc, a], cast(half["grad_out"]).to(dev)
        elif base_name == "WeightedMultiScaleDeformableAttnFunction":
            out = F.apply(v, shapes3, lsi, loc, a, sc, 64)
            leaves, gout = [v, loc, a, sc], cast(half["grad_out"]).to(dev)
        else:
            out = F.apply(d, shapes3, lsi, loc, 64)
            leaves, gout = [d, loc], gscore.to(dev)
        return out, torch.autograd.grad(out, leaves, gout.to(out.dtype))

    with torch.autocast(device_type="cuda", dtype=torch.float16):
        out_t, grads_t = call(twin, lambda x: x)
    out_b, grads_b = call(base, lambda x: x.float())
    assert out_t.dtype == torch.float32
    torch.testing.assert_close(out_t, out_b, rtol=0, atol=0)             # same kernel on the same float32 values
    for gt, gb in zip(grads_t, grads_b):
        assert gt.dtype == torch.float16 and gb.dtype == torch.float32
        torch.testing.assert_close(gt.float(), gb, rtol=2e-3, atol=2e-3)  # float16 rounding of the returned gradient
    # outside autocast the twins take float32 operands unchanged
    out_n, _ = call(twin, lambda x: x.float())
    torch.testing.assert_close(out_n, out_b, rtol=0, atol=0)


def test_bf16_gradients_in_float_buffers_and_in_bf16_buffers_agree(oracle):
    """The C ABI offers bf16 storage with float gradient buffers (DFA3D_BF16) and with bf16 ones (DFA3D_BF16G,
    binned kernels only); the second must be the first rounded to bf16, up to the few rounding adds on shared
    rows, and is refused where the binned kernels do not apply."""
    from dfa3D import _ext, _lib
    from dfa3D.workloads import WORKLOADS, make_inputs, scaled
    dev = _dev()
    inp = make_inputs(scaled(WORKLOADS["base_peaky"], B=2, Q=900), seed=9, device=dev)
    v, d, go = inp["value"].bfloat16(), inp["value_dpt_dist"].bfloat16(), inp["grad_output"].bfloat16()
    sh, lsi, loc, at = (inp[k] for k in ("spatial_shapes", "level_start_index", "sampling_locations", "attention_weights"))
    assert _ext.fused_backward_grad_dtype(v, d, loc) == torch.bfloat16
    res = {}
    for gdt in (torch.float32, torch.bfloat16):
        gv, gd = torch.zeros(v.shape, dtype=gdt, device=dev), torch.zeros(d.shape, dtype=gdt, device=dev)
        gl, ga = torch.empty_like(loc), torch.empty_like(at)
        _ext.dfa3d_fused_backward(v, d, sh, lsi, loc, at, go, None, gv, gd, gl, ga, 64)
        res[gdt] = (gv.float(), gd.float(), gl, ga)
    f, h = res[torch.float32], res[torch.bfloat16]
    torch.testing.assert_close(h[2], f[2], **F32_BWD)
    torch.testing.assert_close(h[3], f[3], **F32_BWD)
    for name, a, b in (("grad_value", h[0], f[0]), ("grad_dist", h[1], f[1])):
        scale = b.abs().max().item()
        torch.testing.assert_close(a, b, rtol=2.0 ** -7, atol=2.0 ** -7 * scale, msg=lambda m, n=name: f"{n}: {m}")
        rel = ((a - b).pow(2).sum() / b.pow(2).sum()).sqrt().item()
        assert rel <= 2.0 ** -8, f"{name}: relative RMS difference {rel:.3g}"
    # an odd number of depth bins: no bf16 gradient buffers, and asking for them anyway is an error, not a fallback
    d_odd = d[..., :63].contiguous()
    sh_odd = sh.clone()
    sh_odd[:, 2] = 63
    assert _ext.fused_backward_grad_dtype(v, d_odd, loc) == torch.float32
    gv, gd = torch.zeros(v.shape, dtype=torch.bfloat16, device=dev), torch.zeros(d_odd.shape, dtype=torch.bfloat16, device=dev)
    with pytest.raises(RuntimeError, match="DFA3D_BF16G"):
        _ext.dfa3d_fused_backward(v, d_odd, sh_odd, lsi, loc, at, go, None, gv, gd, torch.empty_like(loc),
                                  torch.empty_like(at), 64)


@pytest.mark.parametrize("case", [dict(seed=201, B=2, M=4, C=8, D=2, Q=50, P=3, levels=((5, 7), (1, 1), (3, 2))),
                                  dict(seed=202, B=1, M=8, C=32, D=64, Q=400, P=8, levels=((23, 31), (12, 16), (6, 8), (3, 4))),
                                  dict(seed=203, B=3, M=3, C=16, D=17, Q=90, P=5, levels=((9, 4),), lo=-0.6, hi=1.6)],
                         ids=lambda c: f"seed{c['seed']}")
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
def test_packed_shared_distribution_gives_identical_results(oracle, case, dtype):
    """The forward with the distribution packed for its depth taps (dfa3d_pack_dist: one cache line per point
    instead of four) against the forward that gathers from the distribution itself: bit-identical output, scores
    and weight_update, out-of-range locations and one-pixel levels included; and against the checker."""
    from dfa3D import _ext
    dev = _dev()
    t = tiny_case(dtype=torch.float32, **case)
    inp = _as_inputs(t)
    v, d = inp["value"].to(dtype).to(dev), inp["value_dpt_dist"][:, :, :1].contiguous().to(dtype).to(dev)
    sh, lsi = inp["spatial_shapes"].to(dev), inp["level_start_index"].to(dev)
    loc, at = inp["sampling_locations"].to(dev), inp["attention_weights"].to(dev)
    packed = _ext.pack_shared_dist(d, sh, lsi)
    assert packed is not None
    plain = _ext.dfa3d_fused_forward(v, d, sh, lsi, loc, at, 64, need_weight_update=True)
    fast = _ext.dfa3d_fused_forward(v, d, sh, lsi, loc, at, 64, need_weight_update=True, packed_dist=packed)
    for a, b, name in zip(plain, fast, ("output", "depth_score", "weight_update")):
        assert torch.equal(a, b), name
    if dtype == torch.float32:
        shared = dict(inp, value_dpt_dist=inp["value_dpt_dist"][:, :, :1].contiguous())
        want = _shared_dist_expectation(oracle, shared)
        torch.testing.assert_close(fast[0].cpu(), want[0], **F32_FWD)
        torch.testing.assert_close(fast[1].cpu(), want[1], **F32_FWD)
        torch.testing.assert_close(fast[2].cpu(), want[2], **F32_FWD)


def test_packed_distribution_through_the_functions_and_refusals():
    """The weight_update Function takes the packed distribution as an optional eighth argument (one packing for
    several layers) and packs for itself otherwise; both give the gradients of the call without packing.  A single
    depth bin and float64 are not offered; a packed table with a distribution per head is refused."""
    from dfa3D import _ext
    from dfa3D.functional import MultiScale3DDeformableAttnWeightUpdateFunction as F
    from dfa3D.workloads import WORKLOADS, make_inputs, scaled
    dev = _dev()
    inp = make_inputs(scaled(WORKLOADS["base"], B=2, Q=600), seed=21, device=dev)
    sh, lsi = inp["spatial_shapes"], inp["level_start_index"]
    shared = inp["value_dpt_dist"][:, :, :1].contiguous()
    packed = _ext.pack_shared_dist(shared, sh, lsi)
    g = torch.Generator().manual_seed(1)
    gwu = torch.randn(2, 600, 8, 1, generator=g).to(dev)
    results = []
    for extra in ((), (packed,)):
        leaves = [x.clone().requires_grad_() for x in (inp["value"], shared, inp["sampling_locations"], inp["attention_weights"])]
        out, wu = F.apply(leaves[0], leaves[1], sh, lsi, leaves[2], leaves[3], 64, *extra)
        grads = torch.autograd.grad([out, wu], leaves, [inp["grad_output"], gwu])
        results.append((out.detach(), wu.detach(), *grads))
    plain = _ext.dfa3d_fused_forward(inp["value"], shared, sh, lsi, inp["sampling_locations"], inp["attention_weights"], 64,
                                     need_depth_score=False, need_weight_update=True)
    for r in results:
        assert torch.equal(r[0], plain[0]) and torch.equal(r[1], plain[2])
    for a, b in zip(results[0][2:], results[1][2:]):
        torch.testing.assert_close(a, b, **F32_BWD)
    one_bin = shared[..., :1].contiguous()
    assert _ext.pack_shared_dist(one_bin, sh, lsi) is None and _ext.pack_shared_dist(shared.double(), sh, lsi) is None
    with pytest.raises(RuntimeError, match="shared by all heads"):
        _ext.dfa3d_fused_forward(inp["value"], inp["value_dpt_dist"], sh, lsi, inp["sampling_locations"],
                                 inp["attention_weights"], 64, packed_dist=packed)
