"""bench.py's command-line contract: single-GPU only, (on a GPU) one JSON line with the agreed keys, and traffic
figures that are the ones of the committed counter runs of the kernels the library picks."""
import importlib.util
import json
import os
import re
import subprocess
import sys

import pytest

from _util import pkg

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BENCH = os.path.join(ROOT, "bench.py")


def _bench_module():
    spec = importlib.util.spec_from_file_location("cfk_bench", BENCH)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def _counter_row(profile, kernel):
    """(FETCH_SIZE, WRITE_SIZE) in KiB per dispatch: the last two cells of the table row of `profile` whose first cell
    names `kernel` between backticks."""
    rows = [l for l in open(os.path.join(ROOT, profile), encoding="utf-8") if l.startswith("| `" + kernel + "`")]
    assert len(rows) == 1, "%s: %d table rows for %s" % (profile, len(rows), kernel)
    cells = [c.strip() for c in rows[0].strip().strip("|").split("|")]
    return tuple(int(re.sub(r"[ *,]", "", c)) for c in cells[-2:])


def test_traffic_figures_are_those_of_the_committed_counter_runs():
    b = _bench_module()
    cal = b.COPY_CALIBRATION
    assert _counter_row(cal["profile"], cal["kernel"]) == (cal["fetch_kib"], cal["write_kib"])
    for name, t in b.TRAFFIC_SOURCE.items():
        assert _counter_row(t["profile"], t["kernel"]) == (t["fetch_kib"], t["write_kib"]), name
        nbytes, src = b.measured_traffic(name)
        assert src["profile"] == t["profile"] and src["kernel"] == t["kernel"]
        # the scaled figure can only exceed what the algorithm has to move (Q, K, V or A, B read once, the result written once)
        w = b.WORKLOADS[name]
        if w["kind"] == "fmha":
            esz = 1 if w["dtype"] == "f8" else 2
            floor = w["B"] * w["H"] * w["S"] * w["D"] * (3 * esz + 2)
        else:
            floor = 2 * (w["M"] * w["K"] + w["N"] * w["K"] + w["M"] * w["N"])
        assert floor * 0.999 <= nbytes < floor * 8, (name, nbytes, floor)
    assert b.measured_traffic("cfg1") == (None, None)


def test_traffic_figures_name_the_kernel_the_library_picks():
    b = _bench_module()
    f = pkg.fmha
    resource_table = open(os.path.join(ROOT, "profiles", "kernel_resource_usage.md"), encoding="utf-8").read()
    for name, t in b.TRAFFIC_SOURCE.items():
        w = b.WORKLOADS[name]
        if w["kind"] == "fmha":
            dtype = f.CFK_FP8_E4M3 if w["dtype"] == "f8" else f.CFK_FP16
            assert f.fmha_forward_kernel(dtype, w["B"], w["H"], w["S"], w["S"], w["D"]) == t["kernel"], name
        assert "`" + t["kernel"] + "`" in resource_table, name   # ... and it is a kernel of the build


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
    assert rl["traffic"] > 0 and rl["traffic_source"]["profile"].startswith("profiles/") and rl["traffic_source"]["kernel"]
    assert abs(out["value"] - out["config"]["flop_per_step"] / (out["ms_per_step"] * 1e-3) / 1e12) < 1e-6 * out["value"]
    cb = out["cpu_baseline"]
    assert cb["kind"] == "port" and cb["cores"] >= 1 and cb["value"] > 0 and cb["sample"]
