"""bench.py's command-line contract: single-GPU only, and (on a GPU) one JSON line with the agreed keys."""
import json
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BENCH = os.path.join(ROOT, "bench.py")


def test_more_than_one_gpu_is_refused_with_a_message():
    r = subprocess.run([sys.executable, BENCH, "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert r.returncode != 0
    assert "single-GPU" in (r.stdout + r.stderr)


@pytest.mark.gpu
def test_short_run_prints_one_json_line_with_roofline_and_cpu_baseline():
    r = subprocess.run([sys.executable, BENCH, "--steps", "20", "--warmup", "2", "--no-secondary"],
                       capture_output=True, text=True, timeout=600)
    assert r.returncode == 0, r.stdout + r.stderr
    lines = [l for l in r.stdout.splitlines() if l.strip()]
    assert len(lines) == 1
    out = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline"):
        assert key in out, key
    assert out["n_gpus"] == 1 and out["steps"] == 20 and out["warmup"] == 2 and out["vs_baseline"] is None
    assert out["unit"] == "TFLOP/s" and out["dtype"] == "f16" and "workload" in out["config"]
    rl = out["roofline"]
    assert rl["bound"] == "mfma" and rl["peak"] == 2500.0 and abs(rl["frac"] - rl["achieved"] / rl["peak"]) < 1e-9
    assert abs(out["value"] - out["config"]["flop_per_step"] / (out["ms_per_step"] * 1e-3) / 1e12) < 1e-6 * out["value"]
    cb = out["cpu_baseline"]
    assert cb["kind"] == "port" and cb["cores"] >= 1 and cb["value"] > 0 and cb["sample"]
