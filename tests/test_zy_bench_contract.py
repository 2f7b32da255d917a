"""The benchmark's output contract: one JSON line with the agreed keys; more than one GPU is refused."""
import json
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_bench_refuses_more_than_one_gpu():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True,
                       timeout=300)
    assert r.returncode != 0
    assert "--gpus 2" in (r.stdout + r.stderr)


@pytest.mark.gpu
def test_bench_json_line():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--steps", "2", "--warmup", "1", "--no-backward",
                        "--no-layer", "--no-decode"], capture_output=True, text=True, timeout=600)
    assert r.returncode == 0, r.stderr[-2000:]
    lines = [l for l in r.stdout.splitlines() if l.startswith("{")]
    assert len(lines) == 1
    d = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline"):
        assert key in d, key
    assert d["n_gpus"] == 1 and d["steps"] == 2 and d["warmup"] == 1 and d["higher_is_better"] is True
    assert d["vs_baseline"] is None and d["unit"] == "tokens/s" and d["config"]["workload"] == "prefill_cfg4"
    assert abs(d["value"] - 32768 / (d["ms_per_step"] * 1e-3)) <= 1e-6 * d["value"]
    rf = d["roofline"]
    assert rf["bound"] in ("hbm", "mfma") and rf["unit"] in ("GB/s", "TFLOP/s")
    assert rf["achieved"] > 0 and abs(rf["frac"] - rf["achieved"] / rf["peak"]) < 1e-9
    cb = d["cpu_baseline"]
    assert cb["kind"] in ("port", "reference") and cb["value"] > 0 and cb["cores"] >= 1 and cb["sample"]
    # the contracted CPU figure (whole sequence of benchmark configuration 1) next to the sampled one
    c1 = d["cpu_baseline_cfg1"]
    assert c1["kind"] == "port" and c1["value"] > 0 and c1["cores"] >= 1 and "configuration 1" in c1["sample"]
    # the HBM-bound stages and the executed (not only credited) matrix rate of the whole step
    assert d["executed_tflops_whole_step"] >= d["effective_tflops"]
    for name, r in d["roofline_hbm"].items():
        assert r["bound"] == "hbm" and r["unit"] == "GB/s" and r["peak"] == 8000.0 and r["traffic_source"]
        assert (r["traffic"] is None) == (r["achieved"] is None)
        if r["achieved"] is not None:
            assert 0 < r["frac"] <= 1.0
