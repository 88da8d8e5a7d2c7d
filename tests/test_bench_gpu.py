"""bench.py end to end on the GPU: the one JSON line the round's driver reads, with its roofline and CPU baseline."""
import json
import os
import subprocess
import sys

import pytest

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _run(*args):
    p = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), *args], capture_output=True, text=True, timeout=300)
    assert p.returncode == 0, p.stderr[-2000:]
    lines = [l for l in p.stdout.splitlines() if l.strip()]
    assert len(lines) == 1, "bench.py prints exactly one line"
    return json.loads(lines[0])


def test_default_workload_line(gpu_device):
    # (the CPU baseline with one warm-up and one timed iteration per thread count: its keys are what is checked here)
    r = _run("--gpus", "1", "--steps", "5", "--warmup", "2", "--cpu-iters", "1,1")
    assert r["metric"].startswith("MSDA fwd+bwd queries/s") and r["unit"] == "queries/s"
    assert r["n_gpus"] == 1 and r["steps"] == 5 and r["warmup"] == 2
    assert r["higher_is_better"] is True and r["scaling"] == "weak" and r["vs_baseline"] is None
    assert r["dtype"] == "f32" and r["data"] == "synthetic"
    assert r["config"]["workload"].startswith("detr_encoder_bwd") and "model" not in r["config"]
    queries = 2 * 19947
    assert abs(r["value"] - queries / (r["ms_per_step"] * 1e-3)) <= 1e-6 * r["value"]
    assert r["value"] > 0 and r["cold_ms_per_step"] > 0
    assert r["effective_warmup"]["steps_through_autograd"] == 1 + 5 + 2
    assert r["effective_warmup"]["raw_kernel_launches"] >= r["kernels"]["lead_in"]["backward_launches"] > 0
    for key in ("roofline", "roofline_forward", "roofline_backward"):
        f = r[key]
        assert f["bound"] == "hbm" and f["unit"] == "GB/s" and f["peak"] == 8000.0
        assert abs(f["frac"] - f["achieved"] / f["peak"]) < 1e-12 and 0.01 < f["frac"] < 1.0
        assert abs(f["achieved"] - f["algorithmic_bytes"] / (f["kernel_ms"] * 1e-3) / 1e9) <= 1e-6 * f["achieved"]
        # the committed counter figures for this workload: at least the algorithmic bytes, not absurdly more
        assert isinstance(f["traffic"], int) and f["algorithmic_bytes"] <= f["traffic"] < 5 * f["algorithmic_bytes"]
        # (it says where the figure comes from and whether it was measured with the kernel sources of this tree)
        assert f["traffic_from"].startswith("profiles/") and isinstance(f["traffic_measured_with_these_kernel_sources"], bool)
    assert r["roofline"] == r["roofline_backward"]   # the backward is the longer of the two passes
    assert r["roofline_forward"]["algorithmic_bytes"] == 3584 * queries
    assert r["roofline_backward"]["algorithmic_bytes"] == 6144 * queries
    c = r["cpu_baseline"]
    assert c["kind"] == "port" and c["unit"] == "queries/s" and c["cores"] >= 1 and c["value"] > 0 and c["sample"]
    assert c["single_thread"]["cores"] == 1 and c["single_thread"]["value"] > 0
    assert abs(r["speedup_vs_cpu_baseline"] - r["value"] / c["value"]) <= 1e-6 * r["speedup_vs_cpu_baseline"]


def test_other_workload_line_without_committed_traffic(gpu_device):
    r = _run("--workload", "tiny", "--dtype", "float16", "--steps", "3", "--warmup", "1", "--no-cpu-baseline")
    assert r["dtype"] == "f16" and r["config"]["workload"].startswith("tiny")
    assert r["roofline"]["traffic"] is None and "cpu_baseline" not in r
