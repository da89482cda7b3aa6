"""bench.py's command-line contract: more than one GPU is refused with a message,
and a run prints exactly one JSON line carrying the agreed keys."""
import json
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BENCH = os.path.join(ROOT, "bench.py")


def test_more_than_one_gpu_is_refused():
    r = subprocess.run([sys.executable, BENCH, "--gpus", "2"], capture_output=True, text=True, timeout=300)
    assert r.returncode != 0
    assert r.stdout.strip() == ""
    assert "one GPU" in r.stderr


@pytest.mark.gpu
def test_one_json_line_with_the_contract_keys():
    r = subprocess.run([sys.executable, BENCH, "--steps", "20", "--warmup", "3", "--only", "add_f32"],
                       capture_output=True, text=True, timeout=600)
    assert r.returncode == 0, r.stderr[-2000:]
    lines = [l for l in r.stdout.splitlines() if l.strip()]
    assert len(lines) == 1
    d = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline"):
        assert key in d, key
    assert d["n_gpus"] == 1 and d["steps"] == 20 and d["warmup"] == 3 and d["vs_baseline"] is None
    assert d["unit"] == "GB/s" and d["dtype"] == "f32" and d["higher_is_better"] is True
    assert "workload" in d["config"] and "model" not in d["config"]
    roof = d["roofline"]
    assert roof["bound"] == "hbm" and roof["peak"] == 8000.0 and roof["unit"] == "GB/s"
    assert abs(roof["frac"] - roof["achieved"] / roof["peak"]) < 1e-3
    assert abs(d["value"] - roof["achieved"]) < 1e-6
    cpu = d["cpu_baseline"]
    assert cpu["kind"] in ("port", "reference") and cpu["cores"] >= 1 and cpu["value"] > 0 and cpu["sample"]
    # the north star's figures are the last key of the line, each with the copy ceiling measured beside it
    assert list(d)[-1] == "north_star"
    for name in ("layernorm_f32", "add_f32"):
        e = d["north_star"][name]
        assert e["us_per_launch"] > 0 and 0 < e["frac_of_peak"] < 1 and e["copy_ceiling_GBs"] > 0
        assert 0.3 < e["frac_of_copy_ceiling"] < 2.0
    assert d["runner_end_to_end"]["add_f32"]["gpu_runner_us_per_run"] > 0
    # value = algorithmic bytes of one step over the measured time of one step
    assert abs(d["value"] - 25171968 / (d["ms_per_step"] * 1e-3) / 1e9) / d["value"] < 2e-3
