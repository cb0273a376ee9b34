"""The contract of bench.py: one JSON line with the driver's keys, one GPU only."""
import json
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _run(*args, timeout=600):
    return subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), *args], cwd=ROOT, capture_output=True, text=True,
                          timeout=timeout)


def test_more_than_one_gpu_is_refused_with_a_message():
    r = _run("--gpus", "2", "--steps", "1", "--warmup", "0")
    assert r.returncode != 0
    assert "ONE GPU" in r.stderr


@pytest.mark.gpu
def test_one_json_line_with_roofline():
    r = _run("--gpus", "1", "--steps", "20", "--warmup", "5", "--no-cpu", "--layers", "none", "--preheat-ms", "10")
    assert r.returncode == 0, r.stderr[-2000:]
    lines = [l for l in r.stdout.splitlines() if l.strip()]
    assert len(lines) == 1
    d = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "roofline"):   # (cpu_baseline: without --no-cpu)
        assert key in d, key
    assert d["n_gpus"] == 1 and d["steps"] == 20 and d["warmup"] == 5 and d["higher_is_better"] is True
    assert d["vs_baseline"] is None and d["dtype"] == "u8" and d["data"] == "synthetic"
    assert d["config"]["workload"].startswith("C2") and "model" not in d["config"]
    roof = d["roofline"]
    assert roof["bound"] in ("hbm", "mfma") and roof["peak"] == 5000.0
    assert abs(roof["frac"] - roof["achieved"] / roof["peak"]) < 1e-4
    # value = 2 x MACs / time of the timed steps
    assert abs(d["value"] - d["config"]["ops_per_step"] / (d["ms_per_step"] * 1e-3) / 1e12) / d["value"] < 2e-3


@pytest.mark.gpu
def test_chained_network_graph_replay_matches_the_launches():
    r = _run("--network", "mobilenet_v1_int8", "--chained", "--no-cpu", "--preheat-ms", "10")
    assert r.returncode == 0, r.stderr[-2000:]
    d = json.loads([l for l in r.stdout.splitlines() if l.strip()][-1])
    c = d["chained"]
    assert c["graph_replay_matches_eager"] is True
    assert c["eager_ms_per_batch"] > 0 and c["graph_ms_per_batch"] > 0
    assert d["layers_total"] == 28
