"""Builds libdfa3d_hip.so for gfx950 with hipcc (cross-compiles without a GPU).

    python 3d-deformable-attention_amd/build.py [--force]

The library lands next to the python package (dfa3D/libdfa3d_hip.so) so that it travels with
the source tree.
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
MEASURE_LIB = os.path.join(HERE, "dfa3D", "libdfa3d_measure.so")
SOURCES = ["dfa3d_forward.hip", "dfa3d_backward.hip", "dfa3d_backward_binned.hip", "dfa3d_rebatch.hip",
           "dfa3d_api.hip"]
HEADERS = ["dfa3d_device.h", "dfa3d_launch.h", os.path.join("..", "..", "include", "dfa3d.h")]
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


def build(force=False, verbose=True):
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    os.makedirs(OBJ, exist_ok=True)
    deps = [os.path.join(CSRC, h) for h in HEADERS] + [os.path.abspath(__file__)]
    jobs = []
    for src in SOURCES:
        s = os.path.join(CSRC, src)
        o = os.path.join(OBJ, src.replace(".hip", ".o"))
        if force or _stale(o, deps + [s]):
            jobs.append([hipcc, *FLAGS, "-c", s, "-o", o])
    def run(cmd):
        if verbose:
            print(" ".join(cmd), flush=True)
        subprocess.run(cmd, check=True)
    with ThreadPoolExecutor(max_workers=5) as ex:
        list(ex.map(run, jobs))
    objs = [os.path.join(OBJ, s.replace(".hip", ".o")) for s in SOURCES]
    if force or jobs or _stale(LIB, objs):
        run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB, *objs])
    if force or _stale(MEASURE_LIB, [MEASURE_SRC, os.path.join(CSRC, "measure", "dfa3d_measure.h")]):
        run([hipcc, *FLAGS, "-shared", MEASURE_SRC, "-o", MEASURE_LIB])
    return LIB


if __name__ == "__main__":
    build(force="--force" in sys.argv)
    print(LIB)
