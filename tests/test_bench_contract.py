"""The command-line contract of bench.py: one JSON line with the agreed fields; more than one GPU is refused."""
import json
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BENCH = os.path.join(ROOT, "bench.py")


def test_more_than_one_gpu_is_refused_with_a_message():
    out = subprocess.run([sys.executable, BENCH, "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert out.returncode != 0
    assert "ONE GPU" in out.stderr
    assert out.stdout.strip() == ""


@pytest.mark.gpu
def test_one_json_line_with_the_agreed_fields():
    steps, warmup = 3, 1
    out = subprocess.run([sys.executable, BENCH, "--gpus", "1", "--steps", str(steps), "--warmup", str(warmup),
                          "--no-cpu", "--no-configs", "--latency-quick", "--latency-iters", "300"],
                         capture_output=True, text=True, timeout=300)
    assert out.returncode == 0, out.stderr[-2000:]
    lines = [ln for ln in out.stdout.splitlines() if ln.strip()]
    assert len(lines) == 1, lines
    d = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline"):
        assert key in d, key
    assert d["n_gpus"] == 1 and d["steps"] == steps and d["warmup"] == warmup
    assert d["unit"] == "GB/s" and d["higher_is_better"] is True and d["vs_baseline"] is None
    assert d["dtype"] == "f32" and d["data"] == "synthetic" and "workload" in d["config"]
    # value is bytes per step over time per step
    assert d["value"] == pytest.approx(d["config"]["bytes_per_step"] / d["ms_per_step"] / 1e6, rel=1e-3)
    r = d["roofline"]
    for key in ("bound", "achieved", "peak", "unit", "frac", "traffic"):
        assert key in r, key
    assert r["bound"] == "hbm" and r["peak"] == 8000.0 and r["unit"] == "GB/s"
    assert r["frac"] == pytest.approx(r["achieved"] / r["peak"], abs=1e-4)
    assert 0.5 < r["frac"] < 1.0            # below the published peak, and not a broken timer
    if r["traffic"] is not None:            # only reported when the counter summary names this kernel and grid
        assert r["traffic"] == pytest.approx(d["config"]["bytes_per_step"], rel=0.01)
    lat = d["latency_us"]
    for mode in ("sync", "event", "stream", "graph", "issue"):
        assert 0.0 < lat["n4_1024B"][mode]["p50"] <= lat["n4_1024B"][mode]["p99"]
