#!/usr/bin/env python3
"""Benchmark of the DFA3D operator on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload base|small|unit|dense|base_bf16]

A step is one forward + backward of the one-stage autograd Function
(MultiScale3DDeformableAttnFunction.apply -> torch.autograd.grad) over one batch of synthetic
BEVFormer-shaped operands already resident in HBM.  Prints ONE JSON line:

  metric/value   sampled points (B*Q*M*L*P) per second of forward+backward, whole job
  ms_per_step    forward+backward through autograd (includes its allocations and zero fills)
  kernels        launch durations measured with events on the launch stream: the forward kernel, the
                 backward's binning kernels (as a group) and its tile kernel, with the algorithmic
                 GB/s (each operand read once, each result written once) they amount to
  roofline       the same for the dominant (longest) kernel, against MI355X's 8 TB/s HBM peak
  cpu_baseline   the scalar C restatement of the operator (oracle/) on the host cores, on a
                 bounded sample of the same workload
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(ROOT, "3d-deformable-attention_amd"))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0   # MI355X HBM3E, published peak

# HBM-side bytes per launch, from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this script, each
# scaled by what the same counter reads for the library's plain 1 GiB streaming copy (profiles/).
MEASURED_TRAFFIC_BYTES = {
    # profiles/fwd_attention_and_tile_backward_base_fp32.txt
    ("base", "forward"): 5.22e9,
    ("base", "backward_tile"): 4.15e9,
}


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=30)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="base")
    ap.add_argument("--kernel-reps", type=int, default=20, help="launches per kernel for the event timings")
    ap.add_argument("--cpu-seconds", type=float, default=12.0, help="budget of the CPU baseline leg (0 = skip)")
    ap.add_argument("--calibration-copy-mib", type=int, default=0,
                    help="also run one plain streaming copy of this many MiB (yardstick for profiler HBM counters)")
    ap.add_argument("--no-variants", dest="variants", action="store_false",
                    help="skip the timings of the two-stage, shared-distribution and plain-attention entry points")
    ap.add_argument("--tunable", action="append", default=[], metavar="NAME=VALUE", help="library launch tunable")
    return ap.parse_args()


def variant_timings(_ext, torch, value, dist, shapes, lsi, loc, attn, go, reps):
    """Event timings (ms, average) of the other entry points on the same operands: the reference's two-stage
    composition, the caller-shaped call (one distribution for all heads, weight_update instead of the score
    tensor) and plain multi-scale deformable attention (no depth scores)."""
    dev = value.device
    f32 = torch.float32
    out = {}
    score = _ext.ms_depth_score_sample_forward(dist, shapes, lsi, loc, 64)
    gv = torch.zeros(value.shape, dtype=f32, device=dev)
    gd = torch.zeros(dist.shape, dtype=f32, device=dev)
    gl, gl3, ga = torch.empty_like(loc), torch.empty_like(loc), torch.empty_like(attn)
    gs = torch.empty(score.shape, dtype=f32, device=dev)

    def two_stage_fwd():
        sc = _ext.ms_depth_score_sample_forward(dist, shapes, lsi, loc, 64)
        _ext.wms_deform_attn_forward(value, shapes, lsi, loc, attn, sc, 64)

    def two_stage_bwd():
        gv.zero_()
        gd.zero_()
        _ext.wms_deform_attn_backward(value, shapes, lsi, loc, attn, score, go, gv, gl, ga, gs, 64)
        _ext.ms_depth_score_sample_backward(dist, shapes, lsi, loc, gs.to(score.dtype), gd, gl3, 64)

    out["two_stage_fwd_ms"] = round(event_time(two_stage_fwd, reps)[0], 4)
    out["two_stage_bwd_ms"] = round(event_time(two_stage_bwd, reps)[0], 4)
    del score, gs, gl3

    shared = dist[:, :, :1].contiguous()
    gd1 = torch.zeros(shared.shape, dtype=f32, device=dev)

    def shared_bwd():
        gv.zero_()
        gd1.zero_()
        _ext.dfa3d_fused_backward(value, shared, shapes, lsi, loc, attn, go, None, gv, gd1, gl, ga, 64)

    out["shared_dist_weight_update_fwd_ms"] = round(event_time(lambda: _ext.dfa3d_fused_forward(
        value, shared, shapes, lsi, loc, attn, 64, need_depth_score=False, need_weight_update=True), reps)[0], 4)
    out["shared_dist_bwd_ms"] = round(event_time(shared_bwd, reps)[0], 4)

    def plain_bwd():
        gv.zero_()
        _ext.ms_deform_attn_backward(value, shapes, lsi, loc, attn, go, gv, gl, ga, 64)

    out["plain_msda_fwd_ms"] = round(event_time(lambda: _ext.ms_deform_attn_forward(value, shapes, lsi, loc, attn, 64),
                                                reps)[0], 4)
    out["plain_msda_bwd_ms"] = round(event_time(plain_bwd, reps)[0], 4)
    del gv, gd, gd1, gl, ga

    # camera re-batching at BEVFormer-base size: 200x200 BEV queries of 256 channels, 6 cameras that each see
    # a random quarter of them (10 000 per camera: the query count of the operator workload above)
    from dfa3D.rebatch import camera_index, rebatch_combine, rebatch_gather
    g = torch.Generator().manual_seed(0)
    hit = (torch.rand(6, 40000, generator=g) < 0.25).to(dev)
    index, pos, max_len = camera_index(hit)
    bev = torch.randn(1, 40000, 256, generator=g).to(dev)
    scale = (1.0 / hit.sum(0).clamp(min=1).float())[None].contiguous()
    parts = rebatch_gather(bev, index)
    ms_g = event_time(lambda: rebatch_gather(bev, index), reps)[0]
    ms_c = event_time(lambda: rebatch_combine(parts, pos, scale), reps)[0]
    moved = int(hit.sum().item()) * 256 * 4
    out["rebatch_gather_ms"] = round(ms_g, 4)
    out["rebatch_gather_gbs"] = round((moved + parts.numel() * 4) / (ms_g * 1e-3) / 1e9, 1)       # rows read + batch written
    out["rebatch_combine_ms"] = round(ms_c, 4)
    out["rebatch_combine_gbs"] = round((moved + bev.numel() * 4) / (ms_c * 1e-3) / 1e9, 1)        # rows read + slots written
    return out


def event_time(fn, reps, prep=None):
    """Average and minimum duration (ms) of fn() on the current stream, one event pair per call."""
    import torch
    total, best = 0.0, float("inf")
    for _ in range(reps):
        if prep is not None:
            prep()
        s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        s.record()
        fn()
        e.record()
        e.synchronize()
        ms = s.elapsed_time(e)
        total += ms
        best = min(best, ms)
    return total / reps, best


def cpu_baseline(w, budget_s):
    """Forward+backward of the C restatement on a bounded sample (fewer queries, same everything else)."""
    import torch
    from dfa3D.workloads import make_inputs, scaled
    from oracle import dfa3d_oracle as orc
    threads = max(1, min(os.cpu_count() or 1, 64))
    orc.set_threads(threads)
    sample = scaled(w, Q=max(1, min(w.Q, 1000)))
    inp = make_inputs(sample, seed=1234)
    if inp["value"].dtype != torch.float32:
        inp = {k: (v.float() if v.is_floating_point() else v) for k, v in inp.items()}
    args = (inp["value"], inp["value_dpt_dist"], inp["spatial_shapes"], inp["level_start_index"],
            inp["sampling_locations"], inp["attention_weights"])
    reps, spent = 0, 0.0
    while reps < 1 or (spent < budget_s and reps < 50):
        t0 = time.perf_counter()
        _, score = orc.dfa3d_forward(*args)
        orc.dfa3d_backward(*args, score, inp["grad_output"])
        spent += time.perf_counter() - t0
        reps += 1
    per_step = spent / reps
    return {"value": sample.points / per_step, "unit": "points/s", "cores": threads, "kind": "port",
            "sample": f"{w.name} workload with Q={sample.Q} of {w.Q} queries per batch element "
                      f"({sample.points} points), forward+backward, {reps} repetition(s), {per_step * 1e3:.1f} ms each; "
                      f"OpenMP over units (forward) and over the {sample.B} batch elements (backward)"}


def main():
    a = parse()
    if a.gpus != 1:
        print(f"bench.py: this build runs on ONE GPU (one MI355X per box); --gpus {a.gpus} is not supported. "
              "The operator shards over the batch (camera) dimension without any exchange.", file=sys.stderr)
        sys.exit(2)
    import torch
    from dfa3D import _ext, _lib
    from dfa3D.functional import MultiScale3DDeformableAttnFunction
    from dfa3D.workloads import WORKLOADS, make_inputs

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; the HIP kernels are the product and there is no fallback", file=sys.stderr)
        sys.exit(3)
    L_ = _lib.lib()
    for t in a.tunable:
        name, val = t.split("=")
        _lib.set_tunable(name, int(val))

    bf16 = a.workload.endswith("_bf16")
    wname = "base_peaky" if a.workload == "base_bf16" else a.workload
    w = WORKLOADS[wname]
    dev = torch.device("cuda:0")
    inp = make_inputs(w, device=dev)
    value, dist = inp["value"], inp["value_dpt_dist"]
    go = inp["grad_output"]
    if bf16:
        value, dist, go = value.bfloat16(), dist.bfloat16(), go.bfloat16()
    shapes, lsi = inp["spatial_shapes"], inp["level_start_index"]
    loc, attn = inp["sampling_locations"], inp["attention_weights"]
    e_v = 2 if bf16 else 4
    fwd_bytes, bwd_bytes = w.forward_bytes(e_v, e_v), w.backward_bytes(e_v, e_v)

    if a.calibration_copy_mib > 0:
        n = a.calibration_copy_mib << 20
        src = torch.empty(n, dtype=torch.uint8, device=dev).fill_(1)
        dst = torch.empty_like(src)
        for _ in range(2):
            _lib.check(L_.dfa3d_stream_copy(_lib.ptr(dst), _lib.ptr(src), n, _lib.stream_of(src)), "dfa3d_stream_copy")
        torch.cuda.synchronize()
        del src, dst

    leaves = [t.requires_grad_() for t in (value, dist, loc, attn)]

    def step():
        out, _ = MultiScale3DDeformableAttnFunction.apply(leaves[0], leaves[1], shapes, lsi, leaves[2], leaves[3], 64)
        return torch.autograd.grad(out, leaves, go)

    def fwd_only():
        with torch.no_grad():
            return MultiScale3DDeformableAttnFunction.apply(value, dist, shapes, lsi, loc, attn, 64)

    for _ in range(a.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(a.steps):
        step()
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) * 1e3 / a.steps

    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(a.steps):
        fwd_only()
    torch.cuda.synchronize()
    fwd_api_ms = (time.perf_counter() - t0) * 1e3 / a.steps

    # spread of single steps (one event pair each, outside the timed region above)
    singles = []
    for _ in range(max(a.steps, 10)):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        step()
        e1.record()
        e1.synchronize()
        singles.append(e0.elapsed_time(e1))
    singles.sort()
    pick = lambda q: round(singles[min(len(singles) - 1, int(q * len(singles)))], 4)
    step_spread = {"p10": pick(0.1), "median": pick(0.5), "p90": pick(0.9)}

    # ---- per-kernel durations: launches bracketed by events on the launch stream ----
    B, S, M, C = value.shape
    D = dist.shape[3]
    _, Q, _, L, P, _ = loc.shape
    code = _lib.dtype_code(value)
    gv = torch.zeros(value.shape, dtype=torch.float32, device=dev)
    gd = torch.zeros(dist.shape, dtype=torch.float32, device=dev)
    gl = torch.empty_like(loc)
    ga = torch.empty_like(attn)
    vd, dd, ld, ad = value.detach(), dist.detach(), loc.detach(), attn.detach()
    ws_bytes = L_.dfa3d_fused_backward_workspace_bytes(B, S, M, C, D, L, Q, P, dist.shape[2], code)
    ws = torch.empty(max(ws_bytes, 1), dtype=torch.uint8, device=dev)
    stream = _lib.stream_of(value)

    def backward_call():
        _lib.check(L_.dfa3d_fused_backward(
            _lib.ptr(vd), _lib.ptr(dd), _lib.ptr(shapes), _lib.ptr(lsi), _lib.ptr(ld), _lib.ptr(ad), _lib.ptr(go), None,
            None, _lib.ptr(gv), _lib.ptr(gd), _lib.ptr(gl), _lib.ptr(ga), _lib.ptr(ws) if ws_bytes else None, ws_bytes,
            B, S, M, C, D, L, Q, P, dist.shape[2], code, stream), "dfa3d_fused_backward")

    def zero():
        gv.zero_()
        gd.zero_()

    fwd_ms, fwd_best = event_time(lambda: _ext.dfa3d_fused_forward(vd, dd, shapes, lsi, ld, ad, 64), a.kernel_reps)
    bwd_all_ms, bwd_all_best = event_time(backward_call, a.kernel_reps, prep=zero)
    fill_ms, _ = event_time(zero, a.kernel_reps)

    def entry(name, ms, best, nbytes, key=None):
        gbs = nbytes / (ms * 1e-3) / 1e9
        e = {"kernel": name, "avg_ms": round(ms, 4), "min_ms": round(best, 4), "algorithmic_bytes": nbytes,
             "achieved_gbs": round(gbs, 1), "frac_of_hbm_peak": round(gbs / HBM_PEAK_GBS, 4),
             "points_per_s": w.points / (ms * 1e-3)}
        traffic = MEASURED_TRAFFIC_BYTES.get((a.workload, key)) if not bf16 else None
        if traffic:
            # bytes the hardware counters saw on the memory side of the L2, over the time measured here
            e["counter_traffic_gbs"] = round(traffic / (ms * 1e-3) / 1e9, 1)
            e["counter_traffic_frac_of_hbm_peak"] = round(traffic / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)
        return e

    kernels = {"forward": entry("fwd_attention_kernel (depth score + attention, one launch)", fwd_ms, fwd_best, fwd_bytes,
                                "forward")}
    if ws_bytes:
        # binning kernels alone, then the tile kernel alone on the workspace they prepared
        _lib.set_tunable("bwd_stage", 1)
        bin_ms, bin_best = event_time(backward_call, a.kernel_reps)

        def prepare_tile():
            zero()
            _lib.set_tunable("bwd_stage", 1)
            backward_call()
            _lib.set_tunable("bwd_stage", 2)

        tile_ms, tile_best = event_time(backward_call, a.kernel_reps, prep=prepare_tile)
        _lib.set_tunable("bwd_stage", 0)
        kernels["backward_tile"] = entry("tile_backward_kernel (all gradients, one launch)", tile_ms, tile_best, bwd_bytes,
                                         "backward_tile")
        kernels["backward_binning"] = {"kernel": "plan_and_clear + bin_points<0> + bin_scan + bin_points<1> (4 launches)",
                                       "avg_ms": round(bin_ms, 4), "min_ms": round(bin_best, 4)}
        dom = "backward_tile" if tile_ms >= fwd_ms else "forward"
    else:
        kernels["backward_direct"] = entry("bwd_attention_kernel (device-memory atomics)", bwd_all_ms, bwd_all_best, bwd_bytes)
        dom = "backward_direct" if bwd_all_ms >= fwd_ms else "forward"
    k = kernels[dom]
    roofline = {"bound": "hbm", "kernel": k["kernel"], "achieved": k["achieved_gbs"], "peak": HBM_PEAK_GBS,
                "unit": "GB/s", "frac": k["frac_of_hbm_peak"], "traffic": MEASURED_TRAFFIC_BYTES.get((a.workload, dom))}

    result = {
        "metric": "dfa3d_fwd_bwd_sampled_points_per_s",
        "value": w.points / (ms_per_step * 1e-3),
        "unit": "points/s",
        "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16" if bf16 else "f32", "data": "synthetic",
        "config": {"workload": f"{a.workload}: B={w.B} Q={w.Q} M={w.M} C={w.C} L={w.L} "
                               f"levels={'/'.join(f'{h}x{x}' for h, x in w.levels)} D={w.D} P={w.P} "
                               f"({w.points} sampled points), one-stage Function forward+backward"},
        "step_ms_spread": step_spread,
        "fwd_ms": round(fwd_api_ms, 4), "fwd_kernel_ms": round(fwd_ms, 4),
        "bwd_launches_ms": round(bwd_all_ms, 4), "grad_zero_fill_ms": round(fill_ms, 4),
        "fwd_points_per_s": w.points / (fwd_api_ms * 1e-3),
        "fwd_frac_of_hbm_peak": kernels["forward"]["frac_of_hbm_peak"],
        "kernels": kernels,
        "roofline": roofline,
    }
    if a.variants:
        result["variants"] = variant_timings(_ext, torch, vd, dd, shapes, lsi, ld, ad, go, max(a.kernel_reps // 2, 3))
    if a.cpu_seconds > 0:
        result["cpu_baseline"] = cpu_baseline(w, a.cpu_seconds)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
