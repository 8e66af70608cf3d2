"""bench.py prints one JSON line with the agreed keys (run with few steps; the CPU baseline on one head)."""
import json
import os
import subprocess
import sys

import pytest

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_one_json_line_with_roofline_and_cpu_baseline():
    res = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--steps", "3", "--warmup", "1", "--no-extras",
                          "--cpu-heads", "1"], capture_output=True, text=True, timeout=600, cwd=ROOT)
    assert res.returncode == 0, res.stderr[-2000:]
    lines = [ln for ln in res.stdout.splitlines() if ln.strip()]
    assert len(lines) == 1
    d = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline"):
        assert key in d, key
    assert d["n_gpus"] == 1 and d["steps"] == 3 and d["warmup"] == 1 and d["vs_baseline"] is None and d["data"] == "synthetic"
    assert "workload" in d["config"] and "model" not in d["config"]
    r = d["roofline"]
    assert r["bound"] == "mfma" and r["unit"] == "TFLOP/s" and r["peak"] == 2500.0
    assert abs(r["frac"] - r["achieved"] / r["peak"]) < 1e-9 and 0.05 < r["frac"] < 1.0
    c = d["cpu_baseline"]
    assert c["kind"] == "port" and c["cores"] >= 1 and c["value"] > 0 and "sample" in c
    assert d["value"] > c["value"]


def test_more_than_one_gpu_is_refused():
    res = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True,
                         timeout=120, cwd=ROOT)
    assert res.returncode != 0 and "one GPU" in res.stderr


def test_reference_convention_kernel_benchmark_runs():
    """evaluate/bench_kernel.py (the workload and FLOP convention of the reference's script of that name) at a short
    sequence: two JSON lines, forward and backward, with consistent figures."""
    res = subprocess.run([sys.executable, os.path.join(ROOT, "evaluate", "bench_kernel.py"), "--seq", "2048", "--iters", "3"],
                         capture_output=True, text=True, timeout=600, cwd=ROOT)
    assert res.returncode == 0, res.stderr[-2000:]
    rows = [json.loads(ln) for ln in res.stdout.splitlines() if ln.strip()]
    assert [r["mode"] for r in rows] == ["fwd", "bwd"]
    for r in rows:
        assert r["B"] == 2 and r["H"] == 16 and r["L"] == 2048 and r["D"] == 128 and r["BLKQ"] == 128 and r["BLKK"] == 64
        assert r["T"] == 1                                       # min(N, int((1 - 0.95) * N)) with N = 32
        mult = 1.0 if r["mode"] == "fwd" else 2.5
        flops = mult * 4.0 * 2 * 16 * 2048 * 2048 * 128
        assert r["ms"] > 0 and abs(r["effective_tflops"] - flops / r["ms"] * 1e-9) <= 1e-6 * r["effective_tflops"]
    assert 0 < rows[0]["attention_kernel_ms"] <= rows[0]["ms"] * 1.5
