"""bench.py's command-line contract where no GPU is needed: one GPU only, and a loud exit without one."""
import os
import subprocess
import sys

import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _run(*args):
    return subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), *args], capture_output=True, text=True,
                          timeout=300)


def test_more_than_one_gpu_is_refused_with_a_message():
    r = _run("--gpus", "2")
    assert r.returncode != 0 and "ONE GPU" in r.stderr and r.stdout.strip() == ""


def test_no_gpu_no_number():
    if torch.cuda.is_available():
        return
    r = _run("--steps", "1", "--warmup", "0")
    assert r.returncode != 0 and "no fallback" in r.stderr and r.stdout.strip() == ""


def test_recorded_traffic_is_reported_only_for_the_sources_it_was_taken_for(tmp_path, monkeypatch):
    """bench.py takes `roofline.traffic` from profiles/hbm_traffic.json, and only while the kernel sources hash to
    what the file records: a profile of other kernels must read as null, not as a stale figure."""
    import importlib.util
    import json
    spec = importlib.util.spec_from_file_location("bench_under_test", os.path.join(ROOT, "bench.py"))
    bench = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(bench)
    path = tmp_path / "hbm_traffic.json"
    monkeypatch.setattr(bench, "TRAFFIC_JSON", str(path))
    assert bench.recorded_traffic("base")[0] == {}                                   # no file
    entry = {"kernels": {"forward": {"fetch_bytes": 10, "write_bytes": 5}}, "summary": "profiles/x.txt"}
    path.write_text(json.dumps({"base": dict(entry, sources_sha256="0" * 64)}))
    got, why = bench.recorded_traffic("base")
    assert got == {} and "stale" in why
    path.write_text(json.dumps({"base": dict(entry, sources_sha256=bench.sources_digest())}))
    assert bench.recorded_traffic("base")[0] == {"forward": 15}
    assert bench.recorded_traffic("dense")[0] == {}                                  # nothing recorded for that workload


def test_summaries_of_this_scripts_own_json_lines(tmp_path):
    import importlib.util
    import json
    spec = importlib.util.spec_from_file_location("bench_under_test2", os.path.join(ROOT, "bench.py"))
    bench = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(bench)
    run = {"ms_per_step": 3.0, "attainable_gbs": 4700.0,
           "kernels": {"forward": {"avg_ms": 0.9}, "backward_binning": {"avg_ms": 0.3},
                       "backward_tile": {"avg_ms": 1.7, "min_ms": 1.69}}}
    p = tmp_path / "run.json"
    p.write_text(json.dumps(run))
    lines = bench.summarize_json(str(p))
    assert len(lines) == 1 and "tile kernel 1.7000 ms" in lines[0] and "step 3.0000 ms" in lines[0]
