"""Independent statements of what the DFA3D operator computes, used to pin the
CPU checker in ``oracle/``.  None of them shares code or formulas with it.

* ``volume_form``: the operator as a textbook routine.  DFA3D is trilinear
  sampling with zero padding of the expanded volume V[c,d,h,w] =
  value[h,w,c] * dist[h,w,d] (the reference's README.md:18 calls its factorised
  kernels a "mathematically equivalent implementation" of exactly this), i.e.
  ``torch.nn.functional.grid_sample`` on a 5-D input with ``align_corners=False``.
  Differentiable, so ``torch.autograd`` through it gives every gradient.
* ``msda_2d_form``: plain multi-scale deformable attention as 2-D ``grid_sample``;
  the weighted op must reduce to it when every depth score is 1.
* ``brute_*``: python loops straight from the definition, tiny inputs only.
"""
import math

import torch
import torch.nn.functional as F


def tiny_case(seed=0, B=2, M=2, C=3, D=5, Q=7, P=3, levels=((4, 6), (2, 3)), lo=-0.2, hi=1.2,
              dtype=torch.float64, normalise=True):
    g = torch.Generator().manual_seed(seed)
    L = len(levels)
    S = sum(h * w for h, w in levels)
    value = torch.randn(B, S, M, C, generator=g, dtype=dtype)
    dist = torch.randn(B, S, M, D, generator=g, dtype=dtype)
    dist = dist.softmax(-1) if normalise else dist
    loc = torch.rand(B, Q, M, L, P, 3, generator=g, dtype=dtype) * (hi - lo) + lo
    attn = torch.rand(B, Q, M, L * P, generator=g, dtype=dtype).softmax(-1).view(B, Q, M, L, P).contiguous()
    lsi, acc = [], 0
    for h, w in levels:
        lsi.append(acc)
        acc += h * w
    shapes3 = torch.tensor([[h, w, D] for h, w in levels], dtype=torch.int64)
    go = torch.randn(B, Q, M * C, generator=g, dtype=dtype)
    return dict(value=value, dist=dist, loc=loc, attn=attn, shapes3=shapes3,
                lsi=torch.tensor(lsi, dtype=torch.int64), levels=levels, grad_out=go)


def volume_form(value, dist, levels, loc, attn):
    """5-D grid_sample of value (x) dist, weighted by attn, summed over levels and points."""
    B, S, M, C = value.shape
    D = dist.shape[-1]
    Q, P = loc.shape[1], loc.shape[4]
    out = value.new_zeros(B * M, C, Q)
    start = 0
    for l, (H, W) in enumerate(levels):
        v = value[:, start:start + H * W].reshape(B, H, W, M, C).permute(0, 3, 4, 1, 2).reshape(B * M, C, 1, H, W)
        d = dist[:, start:start + H * W].reshape(B, H, W, M, D).permute(0, 3, 4, 1, 2).reshape(B * M, 1, D, H, W)
        start += H * W
        grid = (2 * loc[:, :, :, l] - 1).permute(0, 2, 1, 3, 4).reshape(B * M, Q, P, 1, 3)
        s = F.grid_sample(v * d, grid, mode="bilinear", padding_mode="zeros", align_corners=False)
        a = attn[:, :, :, l].permute(0, 2, 1, 3).reshape(B * M, 1, Q, P)
        out = out + (s.squeeze(-1) * a).sum(-1)
    return out.view(B, M, C, Q).permute(0, 3, 1, 2).reshape(B, Q, M * C)


def msda_2d_form(value, levels, loc_xy, attn):
    """Multi-scale deformable attention as 2-D grid_sample (no depth weighting)."""
    B, S, M, C = value.shape
    Q, P = loc_xy.shape[1], loc_xy.shape[4]
    out = value.new_zeros(B * M, C, Q)
    start = 0
    for l, (H, W) in enumerate(levels):
        v = value[:, start:start + H * W].reshape(B, H, W, M, C).permute(0, 3, 4, 1, 2).reshape(B * M, C, H, W)
        start += H * W
        grid = (2 * loc_xy[:, :, :, l, :, :2] - 1).permute(0, 2, 1, 3, 4).reshape(B * M, Q, P, 2)
        s = F.grid_sample(v, grid, mode="bilinear", padding_mode="zeros", align_corners=False)
        a = attn[:, :, :, l].permute(0, 2, 1, 3).reshape(B * M, 1, Q, P)
        out = out + (s * a).sum(-1)
    return out.view(B, M, C, Q).permute(0, 3, 1, 2).reshape(B, Q, M * C)


def _axis_taps(coord, size):
    """[(index, weight)] of the two linear-interpolation taps along one axis, zero padding."""
    x = coord * size - 0.5
    i0 = math.floor(x)
    t = x - i0
    return [(i, w) for i, w in ((i0, 1.0 - t), (i0 + 1, t)) if 0 <= i < size]


def brute_depth_score(dist, levels, lsi, loc3):
    """Depth score by definition: for each of the four pixels around (x, y), the depth
    distribution of that pixel linearly interpolated at z (zero outside [0, D-1]).
    Returned as a dict keyed by (dh, dw) so that no slot order is assumed."""
    B, S, M, D = dist.shape
    _, Q, _, L, P, _ = loc3.shape
    res = {}
    for b in range(B):
        for q in range(Q):
            for m in range(M):
                for l, (H, W) in enumerate(levels):
                    for p in range(P):
                        x, y, z = (float(t) for t in loc3[b, q, m, l, p])
                        px, py, pz = x * W - 0.5, y * H - 0.5, z * D - 0.5
                        inside = (-1 < px < W) and (-1 < py < H) and (-1 < pz < D)
                        h0, w0 = math.floor(py), math.floor(px)
                        for dh in (0, 1):
                            for dw in (0, 1):
                                hc, wc = h0 + dh, w0 + dw
                                s = 0.0
                                if inside and 0 <= hc < H and 0 <= wc < W:
                                    pix = int(lsi[l]) + hc * W + wc
                                    s = sum(wt * float(dist[b, pix, m, i]) for i, wt in _axis_taps(z, D))
                                res[(b, q, m, l, p, dh, dw)] = s
    return res


def brute_weighted_attention(value, levels, lsi, loc, attn, score_of):
    """out[b,q,m,:] = sum_{l,p} attn * sum_{corner} bilinear(corner) * score(corner) * value[corner];
    ``score_of(b,q,m,l,p,dh,dw)`` supplies the per-corner score."""
    B, S, M, C = value.shape
    _, Q, _, L, P, _ = loc.shape
    out = torch.zeros(B, Q, M, C, dtype=value.dtype)
    for b in range(B):
        for q in range(Q):
            for m in range(M):
                for l, (H, W) in enumerate(levels):
                    for p in range(P):
                        x, y = float(loc[b, q, m, l, p, 0]), float(loc[b, q, m, l, p, 1])
                        px, py = x * W - 0.5, y * H - 0.5
                        if not ((-1 < px < W) and (-1 < py < H)):
                            continue
                        h0, w0 = math.floor(py), math.floor(px)
                        for hc, wy in _axis_taps(y, H):
                            for wc, wx in _axis_taps(x, W):
                                pix = int(lsi[l]) + hc * W + wc
                                out[b, q, m] += (float(attn[b, q, m, l, p]) * wy * wx
                                                 * score_of(b, q, m, l, p, hc - h0, wc - w0) * value[b, pix, m])
    return out.view(B, Q, M * C)


# depth-score slot of the corner (dh, dw): the order the reference stores them in
# (ms_depth_score_sample_cuda_kernel.cuh:89-92): LT, RT, RB, LB
SLOT_OF = {(0, 0): 0, (0, 1): 1, (1, 1): 2, (1, 0): 3}
