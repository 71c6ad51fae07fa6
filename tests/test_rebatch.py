"""Camera re-batching kernels and SpatialCrossAttention_DFA3D against the reference's python-loop form
(BEVFormer_DFA3D/projects/mmdet3d_plugin/bevformer/modules/spatial_cross_attention.py:700-751), restated here
with torch indexing; the inner deformable-attention module is the same object on both sides, so these tests pin
the re-batching alone."""
import copy

import pytest
import torch

LEVELS = ((6, 9), (4, 5))
D = 5


def _mask(cams, bs, Nq, Z, seed=0, p=0.4):
    g = torch.Generator().manual_seed(seed)
    m = torch.rand(cams, bs, Nq, Z, generator=g) < p
    m[1] = False                       # a camera that sees nothing
    m[:, :, 3] = False                 # a query no camera sees
    return m


def test_camera_index_is_the_nonzero_list_and_its_inverse():
    from dfa3D.rebatch import camera_index
    hit = _mask(4, 1, 23, 2)[:, 0].sum(-1) > 0
    index, pos, max_len = camera_index(hit)
    assert index.dtype == torch.int32 and pos.dtype == torch.int32
    assert max_len == int(hit.sum(1).max())
    for i in range(4):
        want = hit[i].nonzero().squeeze(-1)
        assert torch.equal(index[i, :len(want)].long(), want)
        assert (index[i, len(want):] == -1).all()
        assert torch.equal(pos[i][want].long(), torch.arange(len(want)))
        assert (pos[i][~hit[i]] == -1).all()


def _loop_forward(mod, query, key, value, dist, ref_cam, bev_mask, shapes, lsi, query_pos=None):
    """The reference's forward with its loops (:683-751)."""
    inp_residual = query
    slots = torch.zeros_like(query)
    if query_pos is not None:
        query = query + query_pos
    bs, Nq, E = query.shape
    cams = mod.num_cams
    Z = ref_cam.size(3)
    indexes = [m[0].sum(-1).nonzero().squeeze(-1) for m in bev_mask]
    max_len = max(len(e) for e in indexes)
    q_re = query.new_zeros(bs, cams, max_len, E)
    r_re = ref_cam.new_zeros(bs, cams, max_len, Z, 3)
    e_re = query.new_zeros(bs, cams, max_len, mod.num_head, E)
    for j in range(bs):
        for i in range(cams):
            idx = indexes[i]
            q_re[j, i, :len(idx)] = query[j, idx]
            r_re[j, i, :len(idx)] = ref_cam[i][j, idx]
            if mod.use_empty:
                e_re[j, i, :len(idx)] = mod.empty_query.weight.view(mod.bev_h * mod.bev_w, mod.num_head, E)[idx]
    keys = key.shape[1]
    k2 = key.permute(2, 0, 1, 3).reshape(bs * cams, keys, E)
    v2 = value.permute(2, 0, 1, 3).reshape(bs * cams, keys, E)
    d2 = dist.permute(2, 0, 1, 3).reshape(bs * cams, keys, dist.shape[-1])
    out, uw = mod.deformable_attention(query=q_re.view(bs * cams, max_len, E), key=k2, value=v2, value_dpt_dist=d2,
                                       reference_points=r_re.view(bs * cams, max_len, Z, 3), spatial_shapes=shapes,
                                       level_start_index=lsi)
    out = out.view(bs, cams, max_len, E)
    uw = uw.view(bs, cams, *uw.shape[1:])
    if mod.use_empty:
        out = out + ((1 - uw) * e_re).mean(dim=-2)
    for j in range(bs):
        for i, idx in enumerate(indexes):
            slots[j, idx] += out[j, i, :len(idx)]
    count = (bev_mask.sum(-1) > 0).permute(1, 2, 0).sum(-1)
    count = torch.clamp(count, min=1.0)
    slots = slots / count[..., None]
    return mod.dropout(mod.output_proj(slots)) + inp_residual


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float64, torch.float32], ids=["fp64", "fp32"])
def test_gather_and_combine_kernels(dtype):
    from dfa3D.rebatch import RebatchCombineFunction, RebatchGatherFunction, camera_index, rebatch_gather
    dev = torch.device("cuda:0")
    cams, bs, Nq, Z = 4, 3, 37, 2
    for E in (8, 6, 256):                      # 16-byte lanes, scalar lanes, a full embedding row
        g = torch.Generator().manual_seed(E)
        hit = (_mask(cams, 1, Nq, Z, seed=E)[:, 0].sum(-1) > 0).to(dev)
        index, pos, max_len = camera_index(hit)
        src = torch.randn(bs, Nq, E, generator=g, dtype=dtype).to(dev).requires_grad_()
        per_cam = torch.randn(cams, bs, Nq, E, generator=g, dtype=dtype).to(dev)
        scale = torch.rand(bs, Nq, generator=g, dtype=dtype).to(dev)
        got = RebatchGatherFunction.apply(src, index, pos)
        want = src.new_zeros(bs, cams, max_len, E)
        want_pc = src.new_zeros(bs, cams, max_len, E)
        for i in range(cams):
            idx = hit[i].nonzero().squeeze(-1)
            want[:, i, :len(idx)] = src[:, idx]
            want_pc[:, i, :len(idx)] = per_cam[i][:, idx]
        assert torch.equal(got, want.detach())
        assert torch.equal(rebatch_gather(per_cam, index, per_camera=True), want_pc.detach())
        gout = torch.randn(got.shape, generator=g, dtype=dtype).to(dev)
        torch.testing.assert_close(torch.autograd.grad(got, src, gout)[0], torch.autograd.grad(want, src, gout)[0])

        parts = torch.randn(bs, cams, max_len, E, generator=g, dtype=dtype).to(dev).requires_grad_()
        got = RebatchCombineFunction.apply(parts, index, pos, scale)
        want = parts.new_zeros(bs, Nq, E)
        for i in range(cams):
            idx = hit[i].nonzero().squeeze(-1)
            want = want.index_add(1, idx, parts[:, i, :len(idx)])
        want = want * scale[..., None]
        torch.testing.assert_close(got, want.detach())
        gout = torch.randn(got.shape, generator=g, dtype=dtype).to(dev)
        torch.testing.assert_close(torch.autograd.grad(got, parts, gout)[0], torch.autograd.grad(want, parts, gout)[0])


@pytest.mark.gpu
@pytest.mark.parametrize("use_empty", [False, True])
def test_spatial_cross_attention_matches_the_loop_form(use_empty):
    from dfa3D.modules import MSDeformableAttention3D_DFA3D, SpatialCrossAttention_DFA3D
    dev = torch.device("cuda:0")
    torch.manual_seed(5)
    cams, bs, E, heads, Z, bev = 3, 2, 16, 2, 2, 5
    Nq = bev * bev
    attn = MSDeformableAttention3D_DFA3D(embed_dims=E, num_heads=heads, num_levels=len(LEVELS), num_points=4)
    mod = SpatialCrossAttention_DFA3D(embed_dims=E, num_cams=cams, bev_h=bev, bev_w=bev, use_empty=use_empty,
                                      num_head=heads, dropout=0.0, deformable_attention=attn).double()
    with torch.no_grad():
        for p in mod.parameters():
            p.add_(torch.randn_like(p) * 0.2)
    mod = mod.to(dev)
    S = sum(h * w for h, w in LEVELS)
    g = torch.Generator().manual_seed(9)
    f64 = torch.float64
    query = torch.randn(bs, Nq, E, generator=g, dtype=f64).to(dev)
    query_pos = torch.randn(bs, Nq, E, generator=g, dtype=f64).to(dev)
    value = torch.randn(cams, S, bs, E, generator=g, dtype=f64).to(dev)
    dist = torch.randn(cams, S, bs, D, generator=g, dtype=f64).softmax(-1).to(dev)
    ref_cam = torch.rand(cams, bs, Nq, Z, 3, generator=g, dtype=f64).to(dev)
    bev_mask = _mask(cams, bs, Nq, Z, seed=2).to(dev)
    shapes = torch.tensor(LEVELS, dtype=torch.int64, device=dev)
    lsi = torch.tensor([0, 54], dtype=torch.int64, device=dev)

    def run(fn, m):
        leaves = [t.clone().requires_grad_() for t in (query, value, dist)]
        out = fn(m, leaves)
        gout = torch.randn(out.shape, generator=torch.Generator().manual_seed(1), dtype=f64).to(dev)
        grads = torch.autograd.grad(out, leaves + list(m.parameters()), gout, allow_unused=True)
        return out.detach(), grads

    got, got_g = run(lambda m, lv: m(lv[0], lv[1], lv[1], query_pos=query_pos,
                                     spatial_shapes=shapes, reference_points_cam=ref_cam, bev_mask=bev_mask,
                                     level_start_index=lsi, value_dpt_dist=lv[2]), mod)
    ref_mod = copy.deepcopy(mod)
    want, want_g = run(lambda m, lv: _loop_forward(m, lv[0], lv[1], lv[1], lv[2], ref_cam, bev_mask, shapes, lsi,
                                                   query_pos=query_pos), ref_mod)
    tol = dict(rtol=1e-9, atol=1e-10)
    torch.testing.assert_close(got, want, **tol)
    names = ["query", "value", "value_dpt_dist"] + [n for n, _ in mod.named_parameters()]
    for n, a, b in zip(names, got_g, want_g):
        assert (a is None) == (b is None), n
        if a is not None:
            torch.testing.assert_close(a, b, msg=lambda s, n=n: f"grad {n}: {s}", **tol)
