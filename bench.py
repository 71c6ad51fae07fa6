#!/usr/bin/env python3
"""Benchmark of the DFA3D operator on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload base|small|unit|dense|base_bf16|base_f64|unittest|base_coherent]
    python bench.py --micro [xcd]                yardsticks of the machine (copy, bare gathers, LDS atomics, XCD map)
    python bench.py --summarize NAME DIR [DIR..] tables from rocprofv3 output directories -> profiles/NAME.txt
    python bench.py --phase-costs [--workload W] what the parts of the backward's tile kernel cost (development build of
                                                 the library: `python 3d-deformable-attention_amd/build.py --experiment`)

A step is one forward + backward of the one-stage autograd Function
(MultiScale3DDeformableAttnFunction.apply -> torch.autograd.grad) over one batch of synthetic
BEVFormer-shaped operands already resident in HBM.  Prints ONE JSON line:

  metric/value   sampled points (B*Q*M*L*P) per second of forward+backward, whole job
  ms_per_step    forward+backward through autograd (includes its allocations; the backward call clears the part of
                 the gradient buffers that its kernels add to: grad_zero_fill_ms, what zeroing both buffers in
                 full takes, is reported beside it and is no part of a step)
  kernels        launch durations measured with events on the launch stream: the forward kernel, the
                 backward's binning kernels (as a group) and its tile kernel (the library records an event
                 between the two groups of the SAME call), with the algorithmic GB/s (each operand read once,
                 each result written once) they amount to
  roofline       the same for the dominant (longest) kernel, against MI355X's 8 TB/s HBM peak; `traffic` is
                 the HBM-side byte count of that kernel from profiles/hbm_traffic.json when that file was
                 written for the kernel sources as they are now, else null
  roofline_whole_backward   all launches of one backward call against the backward's algorithmic bytes
  attainable_gbs what a plain streaming copy of 1 GiB reaches on this GPU (read + write bytes per second)
  cpu_baseline   the scalar C restatement of the operator (oracle/) on the host cores, on a
                 bounded sample of the same workload
"""
import argparse
import ctypes
import glob
import hashlib
import json
import os
import re
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
PKG = os.path.join(ROOT, "3d-deformable-attention_amd")
sys.path.insert(0, PKG)
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0   # MI355X HBM3E, published peak
TRAFFIC_JSON = os.path.join(ROOT, "profiles", "hbm_traffic.json")
OPTION_NAMES = ("iters", "vec", "direct", "tile", "block", "pass", "chunk")


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="base")
    ap.add_argument("--kernel-reps", type=int, default=20, help="launches per kernel for the event timings")
    ap.add_argument("--cpu-seconds", type=float, default=12.0, help="budget of the CPU baseline leg (0 = skip)")
    ap.add_argument("--calibration-copy-mib", type=int, default=0,
                    help="also run one plain streaming copy of this many MiB (yardstick for profiler HBM counters)")
    ap.add_argument("--no-variants", dest="variants", action="store_false",
                    help="skip the timings of the two-stage, shared-distribution and plain-attention entry points")
    ap.add_argument("--option", action="append", default=[], metavar="NAME=VALUE",
                    help="launch option for every library call (%s)" % ", ".join(OPTION_NAMES))
    ap.add_argument("--micro", nargs="?", const="all", choices=("all", "xcd"),
                    help="run the yardstick kernels instead of the operator (xcd: only the workgroup -> XCD map)")
    ap.add_argument("--phase-costs", action="store_true",
                    help="time the tile kernel of the backward with parts of it cut out, and its per-phase clocks "
                         "(needs libdfa3d_hip_experiment.so; prints a text table)")
    ap.add_argument("--summarize", nargs="+", metavar=("NAME", "DIR"),
                    help="write profiles/NAME.txt (and profiles/hbm_traffic.json) from rocprofv3 output directories")
    ap.add_argument("--summarize-command", action="append", default=[],
                    help="with --summarize: a command line to quote in the summary's header (repeatable)")
    return ap.parse_args()


def sources_digest():
    """SHA-256 over the kernel sources without their comments and blank space: what a traffic figure from the
    profiler is valid for."""
    h = hashlib.sha256()
    for path in sorted(glob.glob(os.path.join(PKG, "csrc", "*.hip")) + glob.glob(os.path.join(PKG, "csrc", "*.h"))):
        text = open(path, encoding="utf-8").read()
        text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
        text = re.sub(r"//[^\n]*", "", text)
        h.update(os.path.basename(path).encode())
        h.update(" ".join(text.split()).encode())
    return h.hexdigest()


def recorded_traffic(workload):
    """{kernel key: HBM-side bytes per launch} from profiles/hbm_traffic.json, or {} when the file is missing,
    holds nothing for this workload or was written for other kernel sources."""
    try:
        doc = json.load(open(TRAFFIC_JSON))
    except (OSError, ValueError):
        return {}, "no profiles/hbm_traffic.json"
    rec = doc.get(workload)
    if not rec:
        return {}, f"profiles/hbm_traffic.json holds nothing for workload {workload}"
    if rec.get("sources_sha256") != sources_digest():
        return {}, "profiles/hbm_traffic.json was written for other kernel sources (stale)"
    return {k: v["fetch_bytes"] + v["write_bytes"] for k, v in rec["kernels"].items()}, rec.get("summary", "")


# ------------------------------------------------------------------------------------------------
# measure library (yardstick kernels)
# ------------------------------------------------------------------------------------------------
def measure_lib():
    path = os.path.join(ROOT, "libdfa3d_measure.so")
    if not os.path.exists(path):
        raise ImportError(f"{path} is missing: build it with `python 3d-deformable-attention_amd/build.py`")
    h = ctypes.CDLL(path)
    P, I, Z = ctypes.c_void_p, ctypes.c_int, ctypes.c_size_t
    h.dfa3d_measure_stream_copy.argtypes = [P, P, Z, P]
    h.dfa3d_measure_xcd_map.argtypes = [P, I, I, I, P]
    h.dfa3d_measure_row_gather.argtypes = [P, Z, I, I, I, I, P, P]
    h.dfa3d_measure_pair_gather.argtypes = [P, Z, I, I, I, P, P]
    h.dfa3d_measure_lds_atomics.argtypes = [I, I, I, P, P]
    return h


def copy_bandwidth(torch, mib=1024, reps=5):
    """GB/s (bytes read + bytes written) of a plain streaming copy: the attainable ceiling on this GPU."""
    m = measure_lib()
    dev = torch.device("cuda:0")
    n = mib << 20
    src = torch.empty(n, dtype=torch.uint8, device=dev).fill_(1)
    dst = torch.empty_like(src)
    stream = ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream)

    def run():
        rc = m.dfa3d_measure_stream_copy(dst.data_ptr(), src.data_ptr(), n, stream)
        assert rc == 0, rc

    run()
    ms, best = event_time(run, reps)
    return 2 * n / (best * 1e-3) / 1e9


def micro(sections="all"):
    """Yardsticks: what the machine does for the bare access patterns of the kernels."""
    import torch
    m = measure_lib()
    dev = torch.device("cuda:0")
    stream = ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream)
    sink = torch.zeros(64, dtype=torch.uint8, device=dev)
    props = torch.cuda.get_device_properties(0)
    cus = props.multi_processor_count
    out = {"device": props.name, "compute_units": cus, "copy_gbs": round(copy_bandwidth(torch), 1)}

    # which XCD do the workgroups of a launch land on?  (the kernels tie heads to XCDs through block id % 8)
    maps = {}
    for blocks, threads in ((4096, 256), (512, 512), (60000, 256)):
        buf = torch.full((blocks,), -1, dtype=torch.int32, device=dev)
        rows = []
        for _ in range(3):
            rc = m.dfa3d_measure_xcd_map(buf.data_ptr(), blocks, threads, 20000, stream)
            assert rc == 0, rc
            torch.cuda.synchronize()
            x = buf.cpu()
            blk = torch.arange(blocks) % 8
            hist = torch.zeros(8, 8, dtype=torch.int64)
            hist.index_put_((blk, x.long().clamp(0, 7)), torch.ones(blocks, dtype=torch.int64), accumulate=True)
            rows.append({"on_diagonal": int(hist.diag().sum()), "blocks": blocks,
                         "xcd_of_block_mod_8": hist.argmax(1).tolist(), "xcds_seen": int(x.unique().numel())})
        maps[f"{blocks}x{threads}"] = rows
    out["xcd_map"] = maps
    if sections == "xcd":
        print(json.dumps(out))
        return

    # random whole-row gathers (the value-row gathers of the forward) against the footprint they are drawn from
    src = torch.zeros(1 << 30, dtype=torch.uint8, device=dev)
    blocks, iters = cus * 32, 64
    rows_tbl = []
    for row_bytes in (128, 256, 64):
        lanes = row_bytes // 16
        for mb in (2, 16, 64, 256, 1024):
            rows = (mb << 20) // row_bytes
            for infl in ((8,) if row_bytes != 128 else (1, 4, 8)):
                fn = lambda: m.dfa3d_measure_row_gather(src.data_ptr(), rows, row_bytes, infl, blocks, iters,
                                                        sink.data_ptr(), stream)
                assert fn() == 0
                _, best = event_time(fn, 3)
                n_rows = blocks * 256 // lanes * iters * infl
                rows_tbl.append({"row_bytes": row_bytes, "footprint_mib": mb, "in_flight": infl,
                                 "tb_per_s": round(n_rows * row_bytes / (best * 1e-3) / 1e12, 2),
                                 "ps_per_row": round(best * 1e-3 / n_rows * 1e12, 1),
                                 "clocks_per_row_per_cu": round(best * 1e-3 / n_rows * cus * 2.4e9, 2)})
    out["row_gather"] = rows_tbl
    # random 8-byte gathers, 64 different lines per wavefront instruction (the depth taps)
    pair_tbl = []
    for mb in (2, 16, 64, 256, 1024):
        for infl in (1, 4, 8):
            fn = lambda: m.dfa3d_measure_pair_gather(src.data_ptr(), mb << 20, infl, blocks, iters, sink.data_ptr(), stream)
            assert fn() == 0
            _, best = event_time(fn, 3)
            n = blocks * 256 * iters * infl
            pair_tbl.append({"footprint_mib": mb, "in_flight": infl, "g_loads_per_s": round(n / (best * 1e-3) / 1e9, 1),
                             "ps_per_load": round(best * 1e-3 / n * 1e12, 1),
                             "clocks_per_load_per_cu": round(best * 1e-3 / n * cus * 2.4e9, 2)})
    out["pair_gather"] = pair_tbl
    del src
    names = ["float add, one bank per lane", "float add, random", "float add, one address",
             "int add returning, random", "int add, random", "int exchange, random"]
    lds = []
    for mode, name in enumerate(names):
        blocks_l, iters_l = 2048, 2000
        fn = lambda: m.dfa3d_measure_lds_atomics(mode, blocks_l, iters_l, sink.data_ptr(), stream)
        assert fn() == 0
        _, best = event_time(fn, 3)
        n = blocks_l * 256 * iters_l
        lds.append({"pattern": name, "lanes_per_clock_per_cu": round(n / (best * 1e-3) / 2.4e9 / cus, 3)})
    out["lds_atomics"] = lds
    print(json.dumps(out))


# ------------------------------------------------------------------------------------------------
# rocprofv3 summaries
# ------------------------------------------------------------------------------------------------
KERNEL_KEYS = (("fwd_attention_kernel", "forward"), ("tile_backward_kernel", "backward_tile"),
               ("cell_backward_kernel", "backward_tile"),
               ("bin_fill_sorted_kernel", "bin_fill"), ("bin_count_kernel", "bin_count"),
               ("bin_scan_kernel", "bin_scan_and_clear"))


def short_name(n):
    n = re.sub(r"\(.*", "", n)
    return n.replace("dfa3d::", "").replace("void ", "").replace("(anonymous namespace)::", "")[:92]


def summarize_json(path):
    """Text form of one JSON line this script printed (a --micro run or an operator run)."""
    doc = json.load(open(path))
    rel = os.path.relpath(path, ROOT)
    out = []
    if "xcd_map" in doc:
        out += ["", f"## {rel}: {doc['device']}, {doc['compute_units']} CUs, plain copy {doc['copy_gbs']} GB/s (read + write)"]
        for launch, rows in doc["xcd_map"].items():
            diag = ", ".join(f"{r['on_diagonal']}/{r['blocks']}" for r in rows)
            out.append(f"workgroup -> XCD, launch of {launch} (workgroups x threads): workgroups with XCD == id % 8: {diag}; "
                       f"XCD of id % 8 = 0..7: {rows[0]['xcd_of_block_mod_8']}")
        if "row_gather" in doc:
            out += ["", "random whole-row gathers (row_bytes/16 lanes per row), by footprint the rows are drawn from",
                    f"{'row_bytes':>9s} {'footprint_MiB':>13s} {'in_flight':>9s} {'TB/s':>7s} {'ps/row':>7s} {'clocks/row/CU':>13s}"]
            out += [f"{r['row_bytes']:9d} {r['footprint_mib']:13d} {r['in_flight']:9d} {r['tb_per_s']:7.2f} {r['ps_per_row']:7.1f} "
                    f"{r['clocks_per_row_per_cu']:13.2f}" for r in doc["row_gather"]]
            out += ["", "random 8-byte loads, one per lane (64 different cache lines per wavefront instruction)",
                    f"{'footprint_MiB':>13s} {'in_flight':>9s} {'G loads/s':>9s} {'ps/load':>7s} {'clocks/load/CU':>14s}"]
            out += [f"{r['footprint_mib']:13d} {r['in_flight']:9d} {r['g_loads_per_s']:9.1f} {r['ps_per_load']:7.1f} "
                    f"{r['clocks_per_load_per_cu']:14.2f}" for r in doc["pair_gather"]]
            out += ["", "LDS atomics, lanes per clock per CU (2.4 GHz)"]
            out += [f"{r['pattern']:32s} {r['lanes_per_clock_per_cu']:7.3f}" for r in doc["lds_atomics"]]
    elif "kernels" in doc:
        k = doc["kernels"]
        out.append(f"{rel}: step {doc['ms_per_step']:.4f} ms, forward kernel {k['forward']['avg_ms']:.4f} ms, "
                   + (f"binning {k['backward_binning']['avg_ms']:.4f} ms, tile kernel {k['backward_tile']['avg_ms']:.4f} ms "
                      f"(min {k['backward_tile']['min_ms']:.4f}), " if "backward_tile" in k else "")
                   + f"copy {doc['attainable_gbs']:.0f} GB/s")
    return out


def source_stamp():
    """What the measured library was built from: the digest of the HIP sources (the same one bench.py checks the
    traffic figures against) and, where git is at hand, the commit with a mark for uncommitted changes."""
    import subprocess
    stamp = f"kernel sources sha256 {sources_digest()[:16]}"
    try:
        head = subprocess.run(["git", "-C", ROOT, "rev-parse", "--short", "HEAD"], capture_output=True, text=True, check=True).stdout.strip()
        dirty = subprocess.run(["git", "-C", ROOT, "status", "--porcelain", "--", "3d-deformable-attention_amd", "bench.py"],
                               capture_output=True, text=True, check=True).stdout.strip()
        stamp += f", git {head}" + (" + uncommitted changes" if dirty else "")
    except (OSError, subprocess.CalledProcessError):
        pass
    return stamp


def summarize(name, dirs, commands):
    """Per-kernel tables from rocprofv3's rocpd databases (kernel durations; counters per dispatch, averaged) as
    text under profiles/, and the HBM-side bytes of the operator's kernels (FETCH_SIZE / WRITE_SIZE, each scaled
    by what the same counter reads for the yardstick copy of known size in the same run) into
    profiles/hbm_traffic.json."""
    import sqlite3
    lines = [f"# {c}" for c in commands] + [f"# {source_stamp()}"]
    scale, raw, workload = {}, {}, None
    for path in [d for d in dirs if d.endswith(".json")]:
        lines += summarize_json(path)
    dirs = [d for d in dirs if not d.endswith(".json")]
    cols = ("fwd_attention_kernel", "cell_backward_kernel", "tile_backward_kernel", "bin_count_kernel",
            "bin_fill_sorted_kernel", "stream_copy_kernel")
    for d in dirs:
        for db in sorted(glob.glob(os.path.join(d, "**", "*.db"), recursive=True)):
            c = sqlite3.connect(db)
            try:
                rows = c.execute("select kernel_name, counter_name, count(*), avg(value) from counters_collection "
                                 "group by kernel_name, counter_name order by 2, 1").fetchall()
            except sqlite3.Error:
                rows = []
            rel = os.path.relpath(db, ROOT)
            if not rows:
                k = c.execute("select name, count(*), avg(end-start), min(end-start), max(end-start), sum(end-start) "
                              "from kernels group by name order by 6 desc").fetchall()
                tot = sum(r[5] for r in k) or 1
                lines += ["", f"## {rel}: kernel durations",
                          f"{'kernel':64s} {'calls':>5s} {'avg_us':>9s} {'min_us':>9s} {'max_us':>9s} {'pct':>5s}"]
                for n, cnt, a, mi, ma, sm in k[:12]:
                    lines.append(f"{short_name(n)[:64]:64s} {cnt:5d} {a / 1e3:9.1f} {mi / 1e3:9.1f} {ma / 1e3:9.1f} {100 * sm / tot:5.1f}")
            else:
                table = {}
                for n, cn, cnt, a in rows:
                    for col in cols:
                        if col in n:
                            table.setdefault(cn, {})[col] = a
                    if "stream_copy_kernel" in n and cn in ("FETCH_SIZE", "WRITE_SIZE"):
                        scale[cn] = a
                    for frag, key in KERNEL_KEYS:
                        if frag in n and cn in ("FETCH_SIZE", "WRITE_SIZE"):
                            raw.setdefault(key, {})[cn] = a
                lines += ["", f"## {rel}: counters, average per dispatch (raw)",
                          f"{'counter':36s} " + " ".join(f"{col[:20]:>20s}" for col in cols)]
                for cn in sorted(table):
                    lines.append(f"{cn:36s} " + " ".join(f"{table[cn].get(col, float('nan')):20.1f}" for col in cols))
            c.close()
    mib = None
    for cmd in commands:
        m = re.search(r"--workload\s+(\S+)", cmd)
        if m:
            workload = m.group(1)
        m = re.search(r"--calibration-copy-mib\s+(\d+)", cmd)
        if m:
            mib = int(m.group(1))
    workload = workload or "base"
    copy_kib = (mib << 10) if mib else None
    traffic = {}
    if copy_kib and "FETCH_SIZE" in scale and "WRITE_SIZE" in scale:
        f_scale, w_scale = copy_kib / scale["FETCH_SIZE"], copy_kib / scale["WRITE_SIZE"]
        lines += ["", f"## HBM-side bytes per launch = counter (KiB) x 1024 x scale factor.  The yardstick copy moves "
                      f"{copy_kib} KiB each way;", f"## FETCH_SIZE reads {scale['FETCH_SIZE']:.0f} for it (factor "
                      f"{f_scale:.3f}), WRITE_SIZE {scale['WRITE_SIZE']:.0f} (factor {w_scale:.3f})"]
        for key, v in raw.items():
            if "FETCH_SIZE" in v and "WRITE_SIZE" in v:
                fb, wb = v["FETCH_SIZE"] * 1024 * f_scale, v["WRITE_SIZE"] * 1024 * w_scale
                traffic[key] = {"fetch_bytes": round(fb), "write_bytes": round(wb)}
                lines.append(f"{key:16s} fetch {fb / 1e9:7.3f} GB   write {wb / 1e9:7.3f} GB   total {(fb + wb) / 1e9:7.3f} GB")
    out_txt = os.path.join(ROOT, "profiles", name + ".txt")
    with open(out_txt, "w") as f:
        f.write("\n".join(lines) + "\n")
    print("wrote", out_txt)
    if traffic:
        try:
            doc = json.load(open(TRAFFIC_JSON))
        except (OSError, ValueError):
            doc = {}
        doc[workload] = {"sources_sha256": sources_digest(), "summary": f"profiles/{name}.txt", "kernels": traffic}
        with open(TRAFFIC_JSON, "w") as f:
            json.dump(doc, f, indent=1, sort_keys=True)
            f.write("\n")
        print("updated", TRAFFIC_JSON)


# ------------------------------------------------------------------------------------------------
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
    packed = _ext.pack_shared_dist(shared, shapes, lsi)
    if packed is not None:     # the same forward with its depth taps from the packed distribution, and the packing itself
        out["shared_dist_packed_fwd_ms"] = round(event_time(lambda: _ext.dfa3d_fused_forward(
            value, shared, shapes, lsi, loc, attn, 64, need_depth_score=False, need_weight_update=True,
            packed_dist=packed), reps)[0], 4)
        out["pack_shared_dist_ms"] = round(event_time(lambda: _ext.pack_shared_dist(shared, shapes, lsi), reps)[0], 4)
    del packed
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


def torch_volume_form_ms(torch, inp, levels, reps=10):
    """Forward of the operator on the CPU with torch.nn.functional.grid_sample on the 5-D volume
    V[c, d, h, w] = value[h, w, c] * dist[h, w, d] (align_corners=False, zero padding), per level."""
    import torch.nn.functional as F
    value, dist, loc, attn = inp["value"], inp["value_dpt_dist"], inp["sampling_locations"], inp["attention_weights"]
    B, S, M, C = value.shape
    D, Q, P = dist.shape[-1], loc.shape[1], loc.shape[4]

    def run():
        out, start = value.new_zeros(B * M, C, Q), 0
        for l, (H, W) in enumerate(levels):
            v = value[:, start:start + H * W].reshape(B, H, W, M, C).permute(0, 3, 4, 1, 2).reshape(B * M, C, 1, H, W)
            d = dist[:, start:start + H * W].reshape(B, H, W, M, D).permute(0, 3, 4, 1, 2).reshape(B * M, 1, D, H, W)
            start += H * W
            grid = (2 * loc[:, :, :, l] - 1).permute(0, 2, 1, 3, 4).reshape(B * M, Q, P, 1, 3)
            s = F.grid_sample(v * d, grid, mode="bilinear", padding_mode="zeros", align_corners=False)
            out = out + (s.squeeze(-1) * attn[:, :, :, l].permute(0, 2, 1, 3).reshape(B * M, 1, Q, P)).sum(-1)
        return out

    with torch.no_grad():
        run()
        t0 = time.perf_counter()
        for _ in range(reps):
            run()
    return (time.perf_counter() - t0) * 1e3 / reps


def cpu_baseline(w, budget_s):
    """Forward+backward of the C restatement on a bounded sample (fewer queries, same everything else)."""
    import torch
    from dfa3D.workloads import WORKLOADS, make_inputs, scaled
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
    # the CPU-sized configuration in full (forward, as the reference's own test would run it)
    unit = make_inputs(WORKLOADS["unit"])
    uargs = (unit["value"], unit["value_dpt_dist"], unit["spatial_shapes"], unit["level_start_index"],
             unit["sampling_locations"], unit["attention_weights"])
    orc.dfa3d_forward(*uargs)
    t0 = time.perf_counter()
    for _ in range(50):
        orc.dfa3d_forward(*uargs)
    unit_ms = (time.perf_counter() - t0) * 1e3 / 50
    # and the same configuration as a user without any extension would run it on these cores: the operator as
    # PyTorch's own trilinear grid_sample of the expanded volume value (x) dist (the equivalence the reference's
    # README.md:18 states), forward only
    torch_ms = torch_volume_form_ms(torch, unit, WORKLOADS["unit"].levels)
    return {"value": sample.points / per_step, "unit": "points/s", "cores": threads, "kind": "port",
            "unit_workload_forward_ms": round(unit_ms, 4),
            "unit_workload_forward_torch_grid_sample_ms": round(torch_ms, 4),
            "unit_workload_forward_points_per_s": WORKLOADS["unit"].points / (unit_ms * 1e-3),
            "sample": f"{w.name} workload with Q={sample.Q} of {w.Q} queries per batch element "
                      f"({sample.points} points), forward+backward, {reps} repetition(s), {per_step * 1e3:.1f} ms each; "
                      f"OpenMP over units (forward) and over the {sample.B} batch elements (backward)"}


# What the development build can cut out of the backward's kernels (dfa3d_experiment_set("diag", bits)), and the
# phases thread 0 of every tile workgroup clocks (-DDFA3D_TILE_TIMING).
PHASE_CUTS = ((0, "nothing (the kernel as shipped, with the phase clocks compiled in)"),
              (16, "the walk of the cells' lists / the task loop of the rows phase (dot products, weighted sums)"),
              (512, "the per-point gradients and grad_dist taps (phase C / finish)"),
              (2, "the grad_dist taps alone"),
              (4, "the flush's device writes"),
              (1, "the LDS tile updates of the rows phase (row-owned kernel only)"),
              (256, "the grad_out row loads"),
              (32, "the depth taps of phase A / prepare"),
              (8, "the value row loads"),
              (1024, "tickets (every grad_dist tap an LDS float atomic)"))
# row-owned kernel (tile_backward_kernel): thread 0's clock, ten slots
PHASE_CLOCKS_ROWS = ("item fetch", "barrier after phases A and C", "rank + staging", "scan + placement", "rows",
                     "phases A and C", "flush", "tail", "-", "-")
# cell-owned kernel (cell_backward_kernel): thread 0 (a walker) fills slots 0-7, thread 256 (a pointer) slots 8-15
PHASE_CLOCKS_CELLS = ("walker: item fetch", "walker: walk (phase X)", "walker: wait at the barrier after X",
                      "walker: stage grad_out rows / hand over accumulators (phase Y)", "walker: wait at the barrier after Y",
                      "-", "-", "walker: flush",
                      "pointer: item fetch", "pointer: late grad_dist taps (phase X)", "pointer: prepare (phase X)",
                      "pointer: wait at the barrier after X", "pointer: place (phase Y)", "pointer: finish (phase Y)",
                      "pointer: wait at the barrier after Y", "pointer: flush")


def phase_costs(a):
    """Text table: tile kernel duration with each part cut out (the difference to the first row is what that part
    costs where it stands), and the share of thread 0's clock each phase takes."""
    import torch
    from dfa3D import _lib
    _lib.LIB_PATH = os.path.join(ROOT, "libdfa3d_hip_experiment.so")
    if not os.path.exists(_lib.LIB_PATH):
        print("bench.py: build the development library first: python 3d-deformable-attention_amd/build.py --experiment",
              file=sys.stderr)
        sys.exit(3)
    from dfa3D.workloads import WORKLOADS, make_inputs
    L_ = _lib.lib()
    L_.dfa3d_experiment_set.argtypes = [ctypes.c_char_p, ctypes.c_int]
    L_.dfa3d_experiment_timer_offset.restype = ctypes.c_size_t
    bf16 = a.workload.endswith("_bf16")
    w = WORKLOADS["base_peaky" if a.workload == "base_bf16" else a.workload]
    dev = torch.device("cuda:0")
    inp = make_inputs(w, device=dev)
    value, dist, go = inp["value"], inp["value_dpt_dist"], inp["grad_output"]
    if bf16:
        value, dist, go = value.bfloat16(), dist.bfloat16(), go.bfloat16()
    shapes, lsi, loc, attn = inp["spatial_shapes"], inp["level_start_index"], inp["sampling_locations"], inp["attention_weights"]
    B, S, M, C = value.shape
    D = dist.shape[3]
    _, Q, _, L, P, _ = loc.shape
    code = _lib.dtype_code(value)
    gv = torch.zeros(value.shape, dtype=torch.float32, device=dev)
    gd = torch.zeros(dist.shape, dtype=torch.float32, device=dev)
    gl, ga = torch.empty_like(loc), torch.empty_like(attn)
    fields = {("pass_" if k == "pass" else k): int(v) for k, v in (t.split("=") for t in a.option)}
    mid = torch.cuda.Event(enable_timing=True)
    mid.record()
    torch.cuda.synchronize()
    opts = ctypes.pointer(_lib.LaunchOptions(event_binned=mid.cuda_event, **fields))
    nbytes = L_.dfa3d_fused_backward_workspace_bytes(B, S, M, C, D, L, Q, P, M, code, opts)
    assert nbytes > 0, "the binned backward does not take this workload"
    ws = torch.zeros(nbytes, dtype=torch.uint8, device=dev)

    def call():
        _lib.check(L_.dfa3d_fused_backward(
            _lib.ptr(value), _lib.ptr(dist), _lib.ptr(shapes), _lib.ptr(lsi), _lib.ptr(loc), _lib.ptr(attn), _lib.ptr(go),
            None, None, _lib.ptr(gv), _lib.ptr(gd), _lib.ptr(gl), _lib.ptr(ga), _lib.ptr(ws), nbytes, B, S, M, C, D, L, Q,
            P, M, code, opts, _lib.stream_of(value)), "dfa3d_fused_backward")

    def timed(reps):
        bins, tiles = [], []
        for i in range(reps + 3):
            gv.zero_()
            gd.zero_()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            call()
            e1.record()
            e1.synchronize()
            if i >= 3:
                bins.append(e0.elapsed_time(mid))
                tiles.append(mid.elapsed_time(e1))
        bins.sort()
        tiles.sort()
        return bins[len(bins) // 2], tiles[len(tiles) // 2]

    print(f"# python bench.py --phase-costs --workload {a.workload}" + "".join(f" --option {t}" for t in a.option))
    print(f"# development build (-DDFA3D_EXPERIMENT -DDFA3D_TILE_TIMING) of the kernel sources with digest {sources_digest()[:16]}")
    print(f"# {torch.cuda.get_device_name(0)}; {w.points} points; medians of {a.kernel_reps} launches; a cut changes results, "
          "its row says what the kernel takes WITHOUT that part")
    print(f"{'cut out':72s} {'binning ms':>10s} {'tile ms':>9s} {'saves ms':>9s}")
    base_tile = None
    for bits, label in PHASE_CUTS:
        L_.dfa3d_experiment_set(b"diag", bits)
        b_ms, t_ms = timed(a.kernel_reps)
        base_tile = t_ms if base_tile is None else base_tile
        print(f"{label:72s} {b_ms:10.4f} {t_ms:9.4f} {base_tile - t_ms:9.4f}", flush=True)
    L_.dfa3d_experiment_set(b"diag", 0)
    gv.zero_()
    gd.zero_()
    ws.zero_()
    call()
    torch.cuda.synchronize()
    off = L_.dfa3d_experiment_timer_offset()
    ticks = ws[off:off + 128].view(torch.int64).cpu().tolist()
    cells = any(ticks[10:])                      # only the cell-owned kernel clocks more than ten slots
    names = PHASE_CLOCKS_CELLS if cells else PHASE_CLOCKS_ROWS
    print("\nshare of a thread's clock per phase, summed over the workgroups of one launch"
          + (" (walkers: wavefronts 0-3, pointers: wavefronts 4-7; each role's shares add up to 100 %)" if cells else ""))
    for lo, hi in ((0, 8), (8, 16)) if cells else ((0, 10),):
        total = sum(ticks[lo:hi]) or 1
        for name, t in zip(names[lo:hi], ticks[lo:hi]):
            if t:
                print(f"{name:72s} {100.0 * t / total:5.1f} %")


def main():
    a = parse()
    if a.summarize:
        summarize(a.summarize[0], a.summarize[1:], a.summarize_command)
        return
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
    if a.micro:
        micro(a.micro)
        return
    if a.phase_costs:
        phase_costs(a)
        return
    L_ = _lib.lib()
    user_options = {}
    for t in a.option:
        name, val = t.split("=")
        if name not in OPTION_NAMES:
            print(f"bench.py: unknown launch option {name}", file=sys.stderr)
            sys.exit(2)
        user_options[name] = int(val)
    with _lib.launch_options(**user_options):
        run(a, torch, _ext, _lib, L_, MultiScale3DDeformableAttnFunction, WORKLOADS, make_inputs, user_options)


def run(a, torch, _ext, _lib, L_, F1, WORKLOADS, make_inputs, user_options):
    bf16, f64 = a.workload.endswith("_bf16"), a.workload.endswith("_f64")
    wname = "base_peaky" if a.workload == "base_bf16" else a.workload[:-4] if f64 else a.workload
    w = WORKLOADS[wname]
    dev = torch.device("cuda:0")
    inp = make_inputs(w, device=dev)
    if f64:         # the other type the reference dispatches (wms_deform_attn_cuda.cu:267): the device-atomics kernels
        inp = {k: (v.double() if v.is_floating_point() else v) for k, v in inp.items()}
    value, dist = inp["value"], inp["value_dpt_dist"]
    go = inp["grad_output"]
    if bf16:
        value, dist, go = value.bfloat16(), dist.bfloat16(), go.bfloat16()
    shapes, lsi = inp["spatial_shapes"], inp["level_start_index"]
    loc, attn = inp["sampling_locations"], inp["attention_weights"]
    e_v = 2 if bf16 else 8 if f64 else 4
    e_a = 8 if f64 else 4
    fwd_bytes, bwd_bytes = w.forward_bytes(e_v, e_v, e_a), w.backward_bytes(e_v, e_v, e_a)

    attainable = copy_bandwidth(torch, mib=max(a.calibration_copy_mib, 1024), reps=5)
    if a.calibration_copy_mib > 0:       # one more copy of exactly the stated size, for the profiler
        copy_bandwidth(torch, mib=a.calibration_copy_mib, reps=1)

    leaves = [t.requires_grad_() for t in (value, dist, loc, attn)]

    def step():
        out, _ = F1.apply(leaves[0], leaves[1], shapes, lsi, leaves[2], leaves[3], 64)
        return torch.autograd.grad(out, leaves, go)

    def fwd_only():
        with torch.no_grad():
            return F1.apply(value, dist, shapes, lsi, loc, attn, 64)

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
    gdt = _ext.fused_backward_grad_dtype(value, dist, loc)          # bf16 storage: the kernel writes bf16 gradients
    code = _lib.DFA3D_BF16G if gdt == torch.bfloat16 else _lib.dtype_code(value)
    gv = torch.zeros(value.shape, dtype=gdt, device=dev)
    gd = torch.zeros(dist.shape, dtype=gdt, device=dev)
    gl = torch.empty_like(loc)
    ga = torch.empty_like(attn)
    vd, dd, ld, ad = value.detach(), dist.detach(), loc.detach(), attn.detach()
    ws_bytes = L_.dfa3d_fused_backward_workspace_bytes(B, S, M, C, D, L, Q, P, dist.shape[2], code, _lib.options())
    ws = torch.empty(max(ws_bytes, 1), dtype=torch.uint8, device=dev)
    stream = _lib.stream_of(value)
    # the library records this event between the binning kernels and the tile kernel of a binned backward
    mid = torch.cuda.Event(enable_timing=True)
    mid.record()
    torch.cuda.synchronize()
    mid_handle = mid.cuda_event
    assert mid_handle, "torch did not create the event"

    user_fields = dict(user_options)
    if "pass" in user_fields:
        user_fields["pass_"] = user_fields.pop("pass")
    # as the autograd Function calls it: gradient buffers not zeroed, the call clears what its kernels add to
    default_opts = ctypes.pointer(_lib.LaunchOptions(clear=1, **user_fields))

    def backward_call(opts=None):
        _lib.check(L_.dfa3d_fused_backward(
            _lib.ptr(vd), _lib.ptr(dd), _lib.ptr(shapes), _lib.ptr(lsi), _lib.ptr(ld), _lib.ptr(ad), _lib.ptr(go), None,
            None, _lib.ptr(gv), _lib.ptr(gd), _lib.ptr(gl), _lib.ptr(ga), _lib.ptr(ws) if ws_bytes else None, ws_bytes,
            B, S, M, C, D, L, Q, P, dist.shape[2], code, opts if opts is not None else default_opts, stream),
            "dfa3d_fused_backward")

    def zero():
        gv.zero_()
        gd.zero_()

    fwd_ms, fwd_best = event_time(lambda: _ext.dfa3d_fused_forward(vd, dd, shapes, lsi, ld, ad, 64), a.kernel_reps)
    bwd_all_ms, bwd_all_best = event_time(backward_call, a.kernel_reps)
    fill_ms, _ = event_time(zero, a.kernel_reps)
    traffic, traffic_note = ({}, "launch options given: recorded traffic does not apply") if user_options \
        else recorded_traffic(a.workload)

    def entry(name, ms, best, nbytes, key=None):
        gbs = nbytes / (ms * 1e-3) / 1e9
        e = {"kernel": name, "avg_ms": round(ms, 4), "min_ms": round(best, 4), "algorithmic_bytes": nbytes,
             "achieved_gbs": round(gbs, 1), "frac_of_hbm_peak": round(gbs / HBM_PEAK_GBS, 4),
             "points_per_s": w.points / (ms * 1e-3)}
        if traffic.get(key):
            # bytes the hardware counters saw on the memory side of the L2: above the algorithmic bytes = lines
            # fetched or written more than once
            e["hbm_side_bytes"] = traffic[key]
            e["hbm_side_bytes_over_algorithmic"] = round(traffic[key] / nbytes, 2)
        return e

    kernels = {"forward": entry("fwd_attention_kernel (depth score + attention, one launch)", fwd_ms, fwd_best, fwd_bytes,
                                "forward")}
    whole_bwd = {"bound": "hbm", "launches": "every kernel of one dfa3d_fused_backward call", "avg_ms": round(bwd_all_ms, 4),
                 "achieved": round(bwd_bytes / (bwd_all_ms * 1e-3) / 1e9, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                 "frac": round(bwd_bytes / (bwd_all_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)}
    if ws_bytes:
        # the two parts of the SAME backward call: [start .. event recorded by the library] = binning kernels,
        # [that event .. end] = tile kernel (plus the head sum for a shared distribution)
        opts = ctypes.pointer(_lib.LaunchOptions(event_binned=mid_handle, clear=1, **user_fields))
        bin_t, tile_t = [], []
        for _ in range(a.kernel_reps):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            backward_call(opts)
            e1.record()
            e1.synchronize()
            bin_t.append(e0.elapsed_time(mid))
            tile_t.append(mid.elapsed_time(e1))
        bin_ms, tile_ms = sum(bin_t) / len(bin_t), sum(tile_t) / len(tile_t)
        kernels["backward_tile"] = entry("tile kernel of the binned backward (all gradients, one launch)", tile_ms, min(tile_t), bwd_bytes,
                                         "backward_tile")
        kernels["backward_binning"] = {"kernel": "plan_and_clear + bin_count + bin_scan (whose further blocks clear gradient rows) + bin_fill_sorted (+ their plain forms, which step aside)",
                                       "avg_ms": round(bin_ms, 4), "min_ms": round(min(bin_t), 4)}
        dom = "backward_tile" if tile_ms >= fwd_ms else "forward"
    else:
        kernels["backward_direct"] = entry("bwd_attention_kernel (device-memory atomics)", bwd_all_ms, bwd_all_best, bwd_bytes)
        dom = "backward_direct" if bwd_all_ms >= fwd_ms else "forward"
    k = kernels[dom]
    roofline = {"bound": "hbm", "kernel": k["kernel"], "achieved": k["achieved_gbs"], "peak": HBM_PEAK_GBS,
                "unit": "GB/s", "frac": k["frac_of_hbm_peak"], "traffic": traffic.get(dom), "traffic_source": traffic_note}

    result = {
        "metric": "dfa3d_fwd_bwd_sampled_points_per_s",
        "value": w.points / (ms_per_step * 1e-3),
        "unit": "points/s",
        "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16" if bf16 else "f64" if f64 else "f32", "data": "synthetic",
        "config": {"workload": f"{a.workload}: B={w.B} Q={w.Q} M={w.M} C={w.C} L={w.L} "
                               f"levels={'/'.join(f'{h}x{x}' for h, x in w.levels)} D={w.D} P={w.P} "
                               f"({w.points} sampled points), one-stage Function forward+backward",
                   "launch_options": user_options},
        "step_ms_spread": step_spread,
        "fwd_ms": round(fwd_api_ms, 4), "fwd_kernel_ms": round(fwd_ms, 4),
        "bwd_launches_ms": round(bwd_all_ms, 4), "grad_zero_fill_ms": round(fill_ms, 4),
        "fwd_points_per_s": w.points / (fwd_api_ms * 1e-3),
        "fwd_frac_of_hbm_peak": kernels["forward"]["frac_of_hbm_peak"],
        "attainable_gbs": round(attainable, 1),
        "kernels": kernels,
        "roofline": roofline,
        "roofline_whole_backward": whole_bwd,
    }
    if a.variants and not f64:
        result["variants"] = variant_timings(_ext, torch, vd, dd, shapes, lsi, ld, ad, go, max(a.kernel_reps // 2, 3))
    if a.cpu_seconds > 0:
        result["cpu_baseline"] = cpu_baseline(w, a.cpu_seconds)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
