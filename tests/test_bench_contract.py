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
