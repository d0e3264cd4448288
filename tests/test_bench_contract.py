"""bench.py's command line and its one JSON line: the keys the driver reads, the roofline and
cpu_baseline objects, and the refusal of more than one GPU."""
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
    assert "one GPU" in r.stderr and "--gpus 1" in r.stderr
    assert r.stdout.strip() == ""                       # no JSON line for a run that did not happen


@pytest.mark.gpu
def test_json_line_has_the_contract_keys():
    r = subprocess.run([sys.executable, BENCH, "--steps", "20", "--warmup", "3", "--no-detail"],
                       capture_output=True, text=True, timeout=600)
    assert r.returncode == 0, r.stderr[-2000:]
    lines = [l for l in r.stdout.splitlines() if l.startswith("{")]
    assert len(lines) == 1, "exactly one JSON line on stdout"
    d = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better",
                "scaling", "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline"):
        assert key in d, key
    assert d["n_gpus"] == 1 and d["steps"] == 20 and d["warmup"] == 3
    assert d["higher_is_better"] is True and d["vs_baseline"] is None and d["data"] == "synthetic"
    assert "workload" in d["config"] and "model" not in d["config"]
    assert abs(d["value"] - 494873344 / (d["ms_per_step"] * 1e-3) / 1e9) < 0.01 * d["value"]   # GB/s = the step's bytes / its time
    rf = d["roofline"]
    for key in ("bound", "achieved", "peak", "unit", "frac", "traffic"):
        assert key in rf, key
    assert rf["bound"] == "hbm" and rf["peak"] == 8000.0 and rf["unit"] == "GB/s"
    assert abs(rf["frac"] - rf["achieved"] / rf["peak"]) < 1e-3 and 0.3 < rf["frac"] < 1.0
    # the launch the step's time goes to, beside the launch its bytes go to, and the step itself
    bt = rf["by_time"]
    for key in ("kernel", "bound", "achieved", "peak", "unit", "frac", "share_of_step", "us_per_launch", "bytes_per_launch"):
        assert key in bt, key
    assert 0.0 < bt["frac"] < 1.0 and 0.0 < bt["share_of_step"] <= 1.0
    assert abs(rf["step"]["frac"] - d["value"] / 8000.0) < 1e-3
    cb = d["cpu_baseline"]
    assert "-O3" in cb["compiler_flags"]
    for key in ("value", "unit", "cores", "kind", "sample"):
        assert key in cb, key
    assert cb["kind"] in ("port", "reference") and cb["cores"] >= 1 and cb["value"] > 0
