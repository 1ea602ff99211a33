"""bench.py: one JSON line with the keys the harness reads; more than one GPU is refused with a message."""
import json
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_more_than_one_gpu_is_refused():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert r.returncode == 2 and "one GPU" in r.stderr and r.stdout.strip() == ""


@pytest.mark.gpu
@pytest.mark.timeout(600)
def test_one_json_line_with_roofline_and_cpu_baseline():
    print("bench contract", flush=True)
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--steps", "3", "--warmup", "1", "--no-extra"],
                       capture_output=True, text=True, timeout=500)
    assert r.returncode == 0, r.stderr[-2000:]
    lines = [l for l in r.stdout.splitlines() if l.strip()]
    assert len(lines) == 1
    d = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline"):
        assert key in d, key
    assert d["n_gpus"] == 1 and d["steps"] == 3 and d["warmup"] == 1 and d["unit"] == "GB/s" and d["vs_baseline"] is None
    assert "workload" in d["config"] and "model" not in d["config"]
    rf = d["roofline"]
    assert rf["bound"] == "hbm" and rf["peak"] == 8000.0 and rf["unit"] == "GB/s"
    assert abs(rf["frac"] - rf["achieved"] / rf["peak"]) < 1e-3 and 0.3 < rf["frac"] < 1.0
    assert rf["traffic"] is None or rf["traffic"] > 0.9 * rf["per_kernel"][rf["kernel"]]["bytes"]
    cb = d["cpu_baseline"]
    assert cb["kind"] == "port" and cb["cores"] >= 1 and cb["value"] > 0 and cb["unit"] == "GB/s" and cb["sample"]
    assert d["value"] > 100 * cb["value"] / 10          # a GPU, not the fallback of anything
    # MX and MoR are both in the timed step; the roofline kernel is the one furthest below the roofline
    pk = rf["per_kernel"]
    assert {"mx_e4m3", "mx_e5m2", "mx_e2m3", "mor_128x128"} <= set(pk)
    assert rf["kernel"] == min(("mx_e4m3", "mx_e5m2", "mx_e2m3", "mor_128x128"), key=lambda k: pk[k]["frac"])
    assert "c1_per_tensor_e4m3_4096x4096" in cb["per_config"]
