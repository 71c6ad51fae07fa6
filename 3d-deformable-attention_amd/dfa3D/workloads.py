"""Synthetic BEVFormer-shaped operands for the DFA3D operator.

Shapes follow what the reference's callers hand to the operator
(unittest_DFA3D.py:43-56 builds the BEVFormer-base case;
BEVFormer_DFA3D/projects/mmdet3d_plugin/bevformer/modules/spatial_cross_attention.py:492-538
builds the operands inside the model).  Every tensor is drawn on the CPU from
one seeded generator in a fixed order (value, depth logits, locations,
attention logits, grad_output) so that a CPU checker and the GPU kernels see
identical bits.
"""
from dataclasses import dataclass, replace
from typing import List, Tuple

import torch


@dataclass(frozen=True)
class Workload:
    name: str
    B: int                      # batch (bs * cameras after re-batching)
    Q: int                      # queries per batch element
    levels: Tuple[Tuple[int, int], ...]   # (H, W) per level
    D: int                      # depth bins
    P: int                      # sampling points per level
    M: int = 8                  # heads
    C: int = 32                 # channels per head
    loc: str = "uniform"        # "uniform" in [lo, hi]^3, "normal" clipped to [lo, hi], "coherent" or "band" (see make_inputs)
    loc_lo: float = 0.0
    loc_hi: float = 1.0
    loc_mean: float = 0.5
    loc_std: float = 0.15
    depth: str = "softmax"      # "softmax" of N(0, sigma) logits or "peaky" (8*onehot + N(0,1))
    depth_sigma: float = 1.0
    attn: str = "softmax"       # "softmax" over levels x points, or "rand": U[0,1) weights that do not sum to 1

    @property
    def L(self):
        return len(self.levels)

    @property
    def S(self):
        return sum(h * w for h, w in self.levels)

    @property
    def points(self):
        return self.B * self.Q * self.M * self.L * self.P

    def level_start_index(self) -> List[int]:
        out, acc = [], 0
        for h, w in self.levels:
            out.append(acc)
            acc += h * w
        return out

    def forward_bytes(self, e_v=4, e_o=4, e_a=4):
        """Algorithmic bytes of one forward: every operand read once, every result written once.  e_v, e_o, e_a:
        bytes per element of value / dist, of output / depth_score, of locations / attention weights."""
        n = self.points
        return (e_v * self.B * self.S * self.M * (self.C + self.D) + 4 * e_a * n + 4 * e_o * n
                + e_o * self.B * self.Q * self.M * self.C)

    def backward_bytes(self, e_v=4, e_o=4, e_a=4):
        """Algorithmic bytes of one backward (saved depth_score re-read, zero fills excluded)."""
        n = self.points
        reads = (e_v * self.B * self.S * self.M * (self.C + self.D) + 4 * e_a * n + 4 * e_o * n
                 + e_o * self.B * self.Q * self.M * self.C)
        writes = e_v * self.B * self.S * self.M * (self.C + self.D) + 4 * e_a * n
        return reads + writes


_BASE_LEVELS = ((116, 200), (58, 100), (29, 50), (15, 25))

WORKLOADS = {
    # the reference-style CPU-runnable case
    "unit": Workload("unit", B=2, Q=100, levels=((16, 16), (8, 8)), D=16, P=4, depth_sigma=1.0),
    # BEVFormer-small style single level, some locations out of bounds
    "small": Workload("small", B=6, Q=4000, levels=((23, 40),), D=64, P=8,
                      loc_lo=-0.05, loc_hi=1.05, depth_sigma=2.0),
    # BEVFormer-base: the headline shape
    "base": Workload("base", B=6, Q=10000, levels=_BASE_LEVELS, D=64, P=8, depth_sigma=2.0),
    # base shape, GT-depth-like peaky distributions (used with bf16 storage)
    "base_peaky": Workload("base_peaky", B=6, Q=10000, levels=_BASE_LEVELS, D=64, P=8, depth="peaky"),
    # the operands of the reference's own test (unittest_DFA3D.py:43-56): 112 depth bins, 9502 queries, attention
    # weights drawn from U[0,1) without normalisation
    "unittest": Workload("unittest", B=6, Q=9502, levels=_BASE_LEVELS, D=112, P=8, attn="rand"),
    # base shape with the locations a trained model produces rather than uniformly random ones: the queries of a
    # camera are BEV pillars in raster order, whose reference points project to a smooth pattern in the image, and
    # the learned offsets move the points of a query by a few pixels around it
    # (spatial_cross_attention.py:505-538: reference point + offset / (W, H, D))
    "base_coherent": Workload("base_coherent", B=6, Q=10000, levels=_BASE_LEVELS, D=64, P=8, depth_sigma=2.0,
                              loc="coherent", loc_std=0.02),
    # Two probes of the forward kernel's cache behaviour at the base shape.  base_coarse: the three coarse levels
    # alone, whose value rows and distributions of one (batch, head) fit an XCD's L2 (2.9 MB).  base_band: all four
    # levels, but the locations of level 0 confined to the upper third of the map, i.e. what a forward that walks
    # level 0 band by band would find in the L2 during one band.
    # base_fine / base_fine_band: level 0 alone (3.84 M points; the tile kernel's work items then all take a single
    # pass), and with its locations confined to that band.
    "base_coarse": Workload("base_coarse", B=6, Q=10000, levels=_BASE_LEVELS[1:], D=64, P=8, depth_sigma=2.0),
    "base_band": Workload("base_band", B=6, Q=10000, levels=_BASE_LEVELS, D=64, P=8, depth_sigma=2.0, loc="band"),
    "base_fine": Workload("base_fine", B=6, Q=10000, levels=_BASE_LEVELS[:1], D=64, P=8, depth_sigma=2.0),
    "base_fine_band": Workload("base_fine_band", B=6, Q=10000, levels=_BASE_LEVELS[:1], D=64, P=8, depth_sigma=2.0,
                               loc="band"),
    # dense BEV grid, clustered locations
    "dense": Workload("dense", B=6, Q=40000, levels=_BASE_LEVELS, D=128, P=8, loc="normal",
                      loc_lo=-0.1, loc_hi=1.1, depth_sigma=2.0),
}

SEEDS = {"unit": 1, "small": 2, "base": 3, "base_peaky": 4, "dense": 5, "unittest": 6, "base_coherent": 7,
         "base_coarse": 3, "base_band": 3, "base_fine": 3, "base_fine_band": 3}


def scaled(w: Workload, B=None, Q=None, name=None) -> Workload:
    """Same distributions and levels with fewer batch elements / queries."""
    return replace(w, B=B or w.B, Q=Q or w.Q, name=name or f"{w.name}[B={B or w.B},Q={Q or w.Q}]")


def make_inputs(w: Workload, seed=None, dtype=torch.float32, device="cpu", grad_output=True):
    """Returns a dict with value, value_dpt_dist, spatial_shapes (L,3), level_start_index,
    sampling_locations (B,Q,M,L,P,3), attention_weights (B,Q,M,L,P) and grad_output."""
    if seed is None:
        seed = SEEDS.get(w.name, 0)
    g = torch.Generator(device="cpu").manual_seed(int(seed))
    B, Q, M, C, L, P, D, S = w.B, w.Q, w.M, w.C, w.L, w.P, w.D, w.S
    value = torch.randn(B, S, M, C, generator=g, dtype=torch.float32)
    if w.depth == "peaky":
        logits = torch.randn(B, S, M, D, generator=g, dtype=torch.float32)
        hot = torch.randint(0, D, (B, S, M, 1), generator=g)
        logits.scatter_add_(-1, hot, torch.full((B, S, M, 1), 8.0))
    else:
        logits = torch.randn(B, S, M, D, generator=g, dtype=torch.float32) * w.depth_sigma
    dist = logits.softmax(-1)
    del logits
    if w.loc == "normal":
        loc = torch.randn(B, Q, M, L, P, 3, generator=g, dtype=torch.float32) * w.loc_std + w.loc_mean
        loc.clamp_(w.loc_lo, w.loc_hi)
    elif w.loc == "coherent":
        # query q sits at cell (q // side, q % side) of a side x side raster over the image; its L*P points per head
        # scatter around that cell's centre with standard deviation loc_std (x, y) and 0.2 around mid-depth (z)
        side = max(1, int(round(Q ** 0.5)))
        q = torch.arange(Q, dtype=torch.float32)
        centre = torch.stack([((q % side) + 0.5) / side, (torch.div(q, side, rounding_mode="floor") % side + 0.5) / side,
                              torch.full((Q,), 0.5)], -1)
        spread = torch.tensor([w.loc_std, w.loc_std, 0.2])
        # (not clipped: a point outside the image is outside the image, as in the model)
        loc = torch.randn(B, Q, M, L, P, 3, generator=g, dtype=torch.float32) * spread + centre.view(1, Q, 1, 1, 1, 3)
    else:
        loc = torch.rand(B, Q, M, L, P, 3, generator=g, dtype=torch.float32) * (w.loc_hi - w.loc_lo) + w.loc_lo
        if w.loc == "band":
            loc[:, :, :, 0, :, 1] /= 3.0                     # level 0: rows of the upper third of the map only
    if w.attn == "rand":
        attn = torch.rand(B, Q, M, L, P, generator=g, dtype=torch.float32)
    else:
        attn = torch.randn(B, Q, M, L * P, generator=g, dtype=torch.float32).softmax(-1).view(B, Q, M, L, P)
    out = {
        "value": value, "value_dpt_dist": dist,
        "spatial_shapes": torch.tensor([[h, w_, D] for h, w_ in w.levels], dtype=torch.int64),
        "level_start_index": torch.tensor(w.level_start_index(), dtype=torch.int64),
        "sampling_locations": loc, "attention_weights": attn.contiguous(),
    }
    if grad_output:
        out["grad_output"] = torch.randn(B, Q, M * C, generator=g, dtype=torch.float32)
    for k, t in out.items():
        if t.is_floating_point():
            t = t.to(dtype)
        out[k] = t.contiguous().to(device)
    return out
