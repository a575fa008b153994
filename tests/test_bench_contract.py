"""bench.py's behaviour that needs no GPU: the refusal of more than one GPU, and the tie between the measured HBM
traffic under profiles/ and the kernel sources it was measured on."""
import json
import os
import subprocess
import sys
import warnings

from conftest import ROOT

sys.path.insert(0, ROOT)
import bench  # noqa: E402


def test_more_than_one_gpu_is_refused_with_a_message():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert r.returncode == 2
    assert "single-GPU" in r.stderr and r.stdout.strip() == ""


def test_traffic_measured_on_other_kernel_sources_is_not_reported(monkeypatch):
    digest = bench.kernel_sources_digest()
    assert len(digest) == 16 and digest == bench.kernel_sources_digest()
    with open(os.path.join(ROOT, "profiles", "hbm_traffic.json")) as f:
        recorded = json.load(f)
    measured, source = bench.load_measured_traffic()
    if recorded.get("_kernel_sources_sha256") == digest:
        assert measured["adam_stream_kernel"]["bytes_per_launch"] >= measured["adam_stream_kernel"]["algorithmic_bytes"]
        assert digest in source and "not measured by this run" in source
    else:
        warnings.warn("profiles/hbm_traffic.json was measured on other kernel sources: bench.py reports no traffic")
        assert measured == {} and "traffic not reported" in source
    monkeypatch.setattr(bench, "kernel_sources_digest", lambda: "0" * 16)
    measured, source = bench.load_measured_traffic()
    assert measured == {} and "traffic not reported" in source


import pytest  # noqa: E402


@pytest.mark.gpu
def test_the_json_line_of_a_small_run():
    """One line of JSON on stdout with the fields the driver reads: the metric and its unit, whole-job value on one
    GPU, steps and warm-up as asked, time per step consistent with the value, the roofline object of the dominant
    kernel (achieved / peak = frac, algorithmic bytes / duration = achieved) and the kernels of a step adding up to
    the step."""
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--small", "--steps", "3", "--warmup", "1",
                        "--no-cpu-baseline", "--no-other-workloads"], capture_output=True, text=True, timeout=600, cwd=ROOT)
    assert r.returncode == 0, r.stderr[-2000:]
    lines = [ln for ln in r.stdout.splitlines() if ln.strip()]
    assert len(lines) == 1
    d = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "roofline"):
        assert key in d, key
    assert d["n_gpus"] == 1 and d["steps"] == 3 and d["warmup"] == 1 and d["higher_is_better"] is True
    assert d["vs_baseline"] is None and d["data"] == "synthetic" and "workload" in d["config"] and "model" not in d["config"]
    roof = d["roofline"]
    assert roof["bound"] == "hbm" and roof["peak"] == 8000.0 and roof["unit"] == "GB/s"
    assert abs(roof["frac"] - roof["achieved"] / roof["peak"]) < 1e-3
    assert abs(roof["achieved"] - roof["algorithmic_bytes_per_launch"] / (roof["ms_per_launch"] * 1e-3) / 1e9) < 0.01 * roof["achieved"]
    assert 0.3 < roof["frac"] < 1.0
    assert roof["traffic"] is None                      # measured for the full-size workload only
    parts = d["other_kernels"]
    step = roof["ms_per_launch"] + parts["has_inf_nan"]["ms"] + parts["ce_forward"]["ms"] + parts["ce_backward"]["ms"]
    assert abs(step - d["ms_per_step"]) < 0.05 * d["ms_per_step"]
