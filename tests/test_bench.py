"""bench.py's command-line contract: one JSON line with the agreed keys on one GPU, a refusal for more."""
import json
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_more_than_one_gpu_is_refused():
    proc = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], cwd=ROOT,
                          stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=120)
    assert proc.returncode != 0 and proc.stdout.strip() == ""
    assert "one GPU" in proc.stderr and "--gpus 2" in proc.stderr


@pytest.mark.gpu
def test_one_json_line_with_the_contract_keys(gpu):
    proc = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--steps", "3", "--warmup", "1",
                           "--cpu-batch", "2"], cwd=ROOT, stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True,
                          timeout=280)
    assert proc.returncode == 0, proc.stderr
    lines = [ln for ln in proc.stdout.splitlines() if ln.strip()]
    assert len(lines) == 1
    d = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline"):
        assert key in d, key
    assert d["n_gpus"] == 1 and d["steps"] == 3 and d["warmup"] == 1 and d["higher_is_better"] is True
    assert d["unit"] == "images/s" and "workload" in d["config"] and "model" not in d["config"]
    assert abs(d["value"] - 256 / (d["ms_per_step"] * 1e-3)) <= 0.01 * d["value"]
    assert abs(d["vs_baseline"] - d["value"] / 5600.0) <= 0.01 * d["vs_baseline"]
    r = d["roofline"]
    for key in ("bound", "achieved", "peak", "unit", "frac", "traffic"):
        assert key in r, key
    assert r["bound"] in ("hbm", "mfma") and abs(r["frac"] - r["achieved"] / r["peak"]) < 1e-3
    c = d["cpu_baseline"]
    for key in ("value", "unit", "cores", "kind", "sample"):
        assert key in c, key
    assert c["kind"] in ("port", "reference") and c["cores"] >= 1
    # the untimed clock-settling passes are reported, and the several-batches-in-flight figure stays out of `value`
    assert d["preheat"]["steps"] >= 8 and d["preheat"]["ms"] > 0
    a = d["as_launched"]
    assert a["unit"] == "images/s" and abs(a["value"] - 256 / (a["ms_per_step"] * 1e-3)) <= 0.01 * a["value"]
    f = d["batches_in_flight"]
    assert f["batches_in_flight"] == 2 and f["unit"] == "images/s" and f["steps"] >= 100
    assert abs(f["value"] - 256 / (f["ms_per_step"] * 1e-3)) <= 0.01 * f["value"]
    assert r["traffic"] is None or r["traffic"] > 0
    assert r["traffic_stale"] == (r["traffic"] is None)
    # the packed first-layer input is a request: its figures stay beside `value`, with the cost of the extra pass
    u = d["packed_input"]
    assert "direct" in u["kernel"] and "direct" not in r["kernel"]
    assert u["pack_ms"] > 0 and u["value_with_pack_in_every_step"] < u["value"]
    assert abs(u["value_with_pack_in_every_step"] - 256e3 / (u["ms_per_step"] + u["pack_ms"])) <= 0.01 * u["value"]
