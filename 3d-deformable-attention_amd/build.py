"""Builds libdfa3d_hip.so for gfx950 with hipcc (cross-compiles without a GPU).

    python 3d-deformable-attention_amd/build.py [--force] [--experiment]

The library lands next to the python package (dfa3D/libdfa3d_hip.so) so that it travels with
the source tree.  Two more libraries land beside bench.py, which is what uses them: the yardstick kernels
(libdfa3d_measure.so) and, with --experiment, libdfa3d_hip_experiment.so: the same sources compiled with
-DDFA3D_EXPERIMENT -DDFA3D_TILE_TIMING, i.e. with the switches that cut parts out of the backward kernels and
the per-phase clocks of the tile kernel (`bench.py --phase-costs`); its results are not the operator's.
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(HERE, "build")
LIB = os.path.join(HERE, "dfa3D", "libdfa3d_hip.so")
# yardstick kernels for bench.py (plain copy, bare gathers, LDS atomics, XCD map): not part of the operator library
MEASURE_SRC = os.path.join(CSRC, "measure", "dfa3d_measure.hip")
ROOT = os.path.dirname(HERE)
MEASURE_LIB = os.path.join(ROOT, "libdfa3d_measure.so")
EXPERIMENT_LIB = os.path.join(ROOT, "libdfa3d_hip_experiment.so")
EXPERIMENT_FLAGS = ["-DDFA3D_EXPERIMENT", "-DDFA3D_TILE_TIMING"]
SOURCES = ["dfa3d_forward.hip", "dfa3d_backward.hip", "dfa3d_backward_binned.hip", "dfa3d_backward_cells.hip",
           "dfa3d_rebatch.hip",
           "dfa3d_api.hip"]
HEADERS = ["dfa3d_device.h", "dfa3d_launch.h", "dfa3d_binned.h", os.path.join("..", "..", "include", "dfa3d.h")]
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-munsafe-fp-atomics",
    # keep the compiler from forming packed fp32 instructions
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function",
]


def _stale(target, deps):
    if not os.path.exists(target):
        return True
    t = os.path.getmtime(target)
    return any(os.path.getmtime(d) > t for d in deps)


def _run(cmd, verbose):
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.run(cmd, check=True)


def _build_lib(lib, obj_dir, extra_flags, force, verbose):
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    os.makedirs(obj_dir, exist_ok=True)
    deps = [os.path.join(CSRC, h) for h in HEADERS] + [os.path.abspath(__file__)]
    jobs = []
    for src in SOURCES:
        s = os.path.join(CSRC, src)
        o = os.path.join(obj_dir, src.replace(".hip", ".o"))
        if force or _stale(o, deps + [s]):
            jobs.append([hipcc, *FLAGS, *extra_flags, "-c", s, "-o", o])
    with ThreadPoolExecutor(max_workers=5) as ex:
        list(ex.map(lambda cmd: _run(cmd, verbose), jobs))
    objs = [os.path.join(obj_dir, s.replace(".hip", ".o")) for s in SOURCES]
    if force or jobs or _stale(lib, objs):
        _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", lib, *objs], verbose)
    return lib


def build(force=False, verbose=True, experiment=False):
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    _build_lib(LIB, OBJ, [], force, verbose)
    if force or _stale(MEASURE_LIB, [MEASURE_SRC, os.path.join(CSRC, "measure", "dfa3d_measure.h")]):
        _run([hipcc, *FLAGS, "-shared", MEASURE_SRC, "-o", MEASURE_LIB], verbose)
    if experiment:
        _build_lib(EXPERIMENT_LIB, os.path.join(OBJ, "experiment"), EXPERIMENT_FLAGS, force, verbose)
    return LIB


if __name__ == "__main__":
    build(force="--force" in sys.argv, experiment="--experiment" in sys.argv)
    print(LIB)
