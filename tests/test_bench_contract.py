"""bench.py's command-line contract: one JSON line with the agreed keys; more than one GPU is refused."""
import json
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_more_than_one_gpu_is_refused_with_a_message():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True,
                       cwd=ROOT, timeout=300)
    assert r.returncode != 0
    assert "one GPU" in (r.stderr + r.stdout) or "1 GPU" in (r.stderr + r.stdout) or "single" in (r.stderr + r.stdout)


@pytest.mark.gpu
def test_default_line_has_the_agreed_keys():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--steps", "10", "--warmup", "2", "--no-e2e"],
                       capture_output=True, text=True, cwd=ROOT, timeout=600)
    assert r.returncode == 0, r.stderr[-2000:]
    lines = [l for l in r.stdout.splitlines() if l.strip()]
    assert len(lines) == 1, lines
    d = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline"):
        assert key in d, key
    assert d["n_gpus"] == 1 and d["steps"] == 10 and d["warmup"] == 2 and d["vs_baseline"] is None
    assert "workload" in d["config"] and "model" not in d["config"]
    roof = d["roofline"]
    for key in ("bound", "achieved", "peak", "unit", "frac", "traffic"):
        assert key in roof, key
    assert roof["bound"] in ("hbm", "mfma") and abs(roof["frac"] - roof["achieved"] / roof["peak"]) < 1e-3
    # the GEMM alone is not slower than quantize + GEMM, and the timed output was checked against the oracle
    assert roof["timing_consistent"] and roof["kernel_us"] <= roof["linear_us"] * 1.01
    assert d["config"]["output_check"]["within_tolerance"] is True
    assert "traffic_source" in roof
    cpu = d["cpu_baseline"]
    for key in ("value", "unit", "cores", "kind", "sample"):
        assert key in cpu, key
    assert cpu["kind"] in ("port", "reference") and cpu["value"] > 0 and d["value"] > 0
