"""MSDeformableAttention3D_DFA3D (the module that calls the operator in DFA3D-BEVFormer's spatial
cross-attention): parameters and initial values as the reference's, and on the GPU the module's outputs and
gradients against a CPU restatement of the reference's forward
(BEVFormer_DFA3D/projects/mmdet3d_plugin/bevformer/modules/spatial_cross_attention.py:472-583) built from
torch layers, the 5-D grid_sample form of the operator and the checker's depth scores."""
import math

import pytest
import torch
import torch.nn.functional as F

from forms import volume_form

LEVELS = ((6, 9), (4, 5), (3, 3))
D = 7


def _module(**kw):
    from dfa3D.modules import MSDeformableAttention3D_DFA3D
    return MSDeformableAttention3D_DFA3D(**kw)


def test_parameters_and_initial_values():
    m = _module(embed_dims=64, num_heads=8, num_levels=3, num_points=4)
    assert sorted(m.state_dict()) == sorted(
        f"{layer}.{p}" for layer in ("sampling_offsets", "sampling_offsets_depth", "attention_weights", "value_proj")
        for p in ("weight", "bias"))
    assert m.sampling_offsets.weight.abs().max() == 0 and m.sampling_offsets_depth.weight.abs().max() == 0
    assert m.attention_weights.weight.abs().max() == 0 and m.attention_weights.bias.abs().max() == 0
    assert m.value_proj.bias.abs().max() == 0
    uv = m.sampling_offsets.bias.view(8, 3, 4, 2)
    dz = m.sampling_offsets_depth.bias.view(8, 3, 4)
    for h in range(8):
        th = 2 * math.pi * h / 8
        c, s = math.cos(th), math.sin(th)
        n = max(abs(c), abs(s))
        for i in range(4):
            want = torch.tensor([c / n, s / n]) * (i + 1)
            assert torch.allclose(uv[h, :, i], want.expand(3, 2), atol=1e-6)
            assert torch.allclose(dz[h, :, i], torch.full((3,), (c + s) / 2 * (i + 1)), atol=1e-6)
    # value projection: Xavier uniform, bound sqrt(6 / (fan_in + fan_out))
    assert m.value_proj.weight.abs().max() <= math.sqrt(6 / 128) + 1e-6
    with pytest.raises(ValueError, match="divisible"):
        _module(embed_dims=30, num_heads=8)


def _inputs(bs=2, Q=5, E=16, Z=2, dtype=torch.float64, seed=0):
    g = torch.Generator().manual_seed(seed)
    S = sum(h * w for h, w in LEVELS)
    query = torch.randn(bs, Q, E, generator=g, dtype=dtype)
    value = torch.randn(bs, S, E, generator=g, dtype=dtype)
    dist = torch.randn(bs, S, D, generator=g, dtype=dtype).softmax(-1)
    ref = torch.rand(bs, Q, Z, 3, generator=g, dtype=dtype)
    shapes = torch.tensor(LEVELS, dtype=torch.int64)
    lsi = torch.tensor([0, 54, 74], dtype=torch.int64)
    go = torch.randn(bs, Q, E, generator=g, dtype=dtype)
    return query, value, dist, ref, shapes, lsi, go


def _randomise(m, seed=1):
    g = torch.Generator().manual_seed(seed)
    with torch.no_grad():
        for p in m.parameters():
            p.add_(torch.randn(p.shape, generator=g, dtype=p.dtype) * 0.3)
    return m


def _restated_forward(m, query, value, dist, ref, shapes):
    """The reference's forward, line by line in torch, with the operator as value (x) dist grid_sample."""
    bs, Q, _ = query.shape
    S = value.shape[1]
    M, L, P = m.num_heads, m.num_levels, m.num_points
    v = F.linear(value, m.value_proj.weight, m.value_proj.bias).view(bs, S, M, -1)
    d = dist.view(bs, S, 1, D).repeat(1, 1, M, 1)
    uv = F.linear(query, m.sampling_offsets.weight, m.sampling_offsets.bias).view(bs, Q, M, L, P, 2)
    dz = F.linear(query, m.sampling_offsets_depth.weight, m.sampling_offsets_depth.bias).view(bs, Q, M, L, P, 1)
    off = torch.cat([uv, dz], -1)
    att = F.linear(query, m.attention_weights.weight, m.attention_weights.bias).view(bs, Q, M, L * P).softmax(-1)
    att = att.view(bs, Q, M, L, P)
    shapes3 = torch.cat([shapes, torch.full((L, 1), D, dtype=shapes.dtype)], -1)
    normalizer = torch.stack([shapes3[:, 1], shapes3[:, 0], shapes3[:, 2]], -1).to(query.dtype)
    Z = ref.shape[2]
    off = (off / normalizer[None, None, None, :, None, :]).view(bs, Q, M, L, P // Z, Z, 3)
    loc = (ref[:, :, None, None, None, :, :] + off).view(bs, Q, M, L, P, 3)
    return volume_form(v, d, LEVELS, loc, att), v, d, loc, att, shapes3


def test_sampling_locations_follow_the_reference_layout():
    m = _randomise(_module(embed_dims=16, num_heads=2, num_levels=3, num_points=4).double())
    query, value, dist, ref, shapes, lsi, _ = _inputs()
    _, _, _, loc, _, shapes3 = _restated_forward(m, query, value, dist, ref, shapes)
    got = m.sampling_locations(query, ref, m.get_spatial_shape_3D(shapes, D))
    assert torch.equal(m.get_spatial_shape_3D(shapes, D), shapes3)
    torch.testing.assert_close(got, loc, rtol=1e-12, atol=1e-12)
    with pytest.raises(ValueError, match="reference_points"):
        m.sampling_locations(query, ref[..., :2], shapes3)
    with pytest.raises(NotImplementedError):
        m(query, value=value, value_dpt_dist=dist, reference_points=ref, spatial_shapes=shapes, level_start_index=lsi)


@pytest.mark.gpu
@pytest.mark.parametrize("batch_first", [True, False])
def test_module_matches_restated_reference_forward_and_gradients(oracle, batch_first):
    dev = torch.device("cuda:0")
    m = _randomise(_module(embed_dims=16, num_heads=2, num_levels=3, num_points=4, batch_first=batch_first).double())
    query, value, dist, ref, shapes, lsi, go = _inputs()
    cpu_leaves = [t.clone().requires_grad_() for t in (query, value, dist)]
    want_out, v, d, loc, att, shapes3 = _restated_forward(m, *cpu_leaves, ref, shapes)
    score = oracle.depth_score_forward(d.detach().contiguous(), shapes3, lsi, loc.detach().contiguous())
    want_wu = (score.mean(-1) * att.detach()).flatten(-2).sum(-1, keepdim=True)
    params = list(m.parameters())
    want_grads = torch.autograd.grad(want_out, cpu_leaves + params, go)

    import copy
    mg = copy.deepcopy(m).to(dev)
    gpu_leaves = [t.to(dev).requires_grad_() for t in (query, value, dist)]
    q_in, v_in = (gpu_leaves[0], gpu_leaves[1]) if batch_first else (gpu_leaves[0].permute(1, 0, 2),
                                                                     gpu_leaves[1].permute(1, 0, 2))
    out, wu, sc = mg(q_in, value=v_in, value_dpt_dist=gpu_leaves[2], reference_points=ref.to(dev),
                     spatial_shapes=shapes.to(dev), level_start_index=lsi.to(dev), return_depth_score=True)
    out2, wu2 = mg(q_in, value=v_in, value_dpt_dist=gpu_leaves[2], reference_points=ref.to(dev),
                   spatial_shapes=shapes.to(dev), level_start_index=lsi.to(dev))
    out_bf = out if batch_first else out.permute(1, 0, 2)
    tol = dict(rtol=1e-9, atol=1e-10)
    torch.testing.assert_close(out_bf.detach().cpu(), want_out.detach(), **tol)
    torch.testing.assert_close(sc.detach().cpu(), score, **tol)
    torch.testing.assert_close(wu.detach().cpu(), want_wu, **tol)
    torch.testing.assert_close(wu2.detach().cpu(), want_wu, **tol)
    torch.testing.assert_close(out2.detach().cpu(), out.detach().cpu(), rtol=0, atol=0)
    out2_bf = out2 if batch_first else out2.permute(1, 0, 2)
    got_grads = torch.autograd.grad(out2_bf, gpu_leaves + list(mg.parameters()), go.to(dev))
    names = ["query", "value", "value_dpt_dist"] + [n for n, _ in m.named_parameters()]
    for n, g_, w_ in zip(names, got_grads, want_grads):
        torch.testing.assert_close(g_.cpu(), w_, msg=lambda s, n=n: f"grad {n}: {s}", **tol)


@pytest.mark.gpu
def test_module_with_a_distribution_packed_once_for_several_calls():
    """float32 module: the packed distribution handed in (as an encoder with several layers on one distribution
    would) gives the output and weight_update of the call that packs for itself, bit for bit, and gradients."""
    dev = torch.device("cuda:0")
    m = _randomise(_module(embed_dims=16, num_heads=2, num_levels=3, num_points=4)).to(dev)
    query, value, dist, ref, shapes, lsi, go = (t.to(dev) if torch.is_tensor(t) else t for t in _inputs(dtype=torch.float32))
    kw = dict(value=value, value_dpt_dist=dist, reference_points=ref, spatial_shapes=shapes, level_start_index=lsi)
    packed = m.pack_dist(dist, shapes, lsi)
    assert packed is not None
    q = query.clone().requires_grad_()
    out1, wu1 = m(q, **kw)
    out2, wu2 = m(q, packed_dist=packed, **kw)
    out3, wu3 = m(q, packed_dist=packed, **kw)             # the same packed tensor again
    assert torch.equal(out1, out2) and torch.equal(wu1, wu2) and torch.equal(out2, out3)
    g1, = torch.autograd.grad(out1, q, go, retain_graph=True)
    g2, = torch.autograd.grad(out2, q, go)
    torch.testing.assert_close(g1, g2, rtol=1e-5, atol=1e-6)
