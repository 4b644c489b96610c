"""The benchmark's command line: one JSON line with the agreed keys, one GPU only."""
import json
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
pytestmark = pytest.mark.gpu


def _run(*args):
    return subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), *args], cwd=ROOT, capture_output=True, text=True,
                          timeout=110)


def test_bench_prints_one_json_line_with_the_agreed_keys():
    r = _run("--workload", "cfg1", "--steps", "3", "--warmup", "1", "--no-cpu")
    assert r.returncode == 0, r.stderr[-2000:]
    lines = [ln for ln in r.stdout.splitlines() if ln.strip()]
    assert len(lines) == 1
    line = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline"):
        assert key in line, key
    assert line["n_gpus"] == 1 and line["steps"] == 3 and line["warmup"] == 1
    assert line["vs_baseline"] is None and line["dtype"] == "f32" and "workload" in line["config"]
    roof = line["roofline"]
    for key in ("bound", "achieved", "peak", "unit", "frac", "traffic"):
        assert key in roof, key
    assert roof["peak"] == 8000.0 and abs(roof["frac"] - roof["achieved"] / roof["peak"]) < 1e-3
    assert line["value"] > 0 and abs(line["value"] - 2 * line["config"]["voxels"] / (line["ms_per_step"] * 1e-3)) < 1e-6 * line["value"]


def test_bench_refuses_more_than_one_gpu():
    r = _run("--gpus", "2")
    assert r.returncode != 0
    assert "one GPU" in r.stderr
