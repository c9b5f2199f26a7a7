"""bench.py's command-line contract: one JSON line with the agreed keys on one GPU, a refusal for more."""
import json
import os
import subprocess
import sys

import pytest
import torch

from conftest import ROOT

BENCH = os.path.join(ROOT, "bench.py")


def test_more_than_one_gpu_is_refused_with_a_message():
    proc = subprocess.run([sys.executable, BENCH, "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert proc.returncode != 0
    assert "one GPU" in proc.stderr and proc.stdout.strip() == ""


@pytest.mark.gpu
def test_one_json_line_with_roofline_and_cpu_baseline():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    proc = subprocess.run([sys.executable, BENCH, "--config", "cfg2", "--steps", "3", "--warmup", "1"],
                          capture_output=True, text=True, timeout=600)
    assert proc.returncode == 0, proc.stderr[-2000:]
    lines = [l for l in proc.stdout.splitlines() if l.strip()]
    assert len(lines) == 1
    d = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline"):
        assert key in d, key
    assert d["n_gpus"] == 1 and d["steps"] == 3 and d["warmup"] == 1 and d["higher_is_better"] is True
    assert d["unit"] == "tokens/s" and d["vs_baseline"] is None and d["data"] == "synthetic" and d["dtype"] == "f32"
    assert "workload" in d["config"] and "model" not in d["config"]
    r = d["roofline"]
    assert r["bound"] == "hbm" and r["unit"] == "GB/s" and r["peak"] == 8000.0      # groups of 4 rows: bandwidth-bound
    assert abs(r["frac"] - r["achieved"] / r["peak"]) < 1e-12 and "traffic" in r
    assert r["valu_achieved_TFLOPs"] > 0 and r["hbm_achieved_GBps"] == r["achieved"]
    assert d["stack"]["min_ms_per_step"] <= d["stack"]["median_ms_per_step"] <= d["stack"]["max_ms_per_step"]
    assert "B=4096 D=1024 g=4" in d["metric"]
    c = d["cpu_baseline"]
    assert c["kind"] in ("reference", "port") and c["cores"] >= 1 and c["value"] > 0 and c["sample"]
    assert abs(d["value"] - 32 * 128 / (d["ms_per_step"] * 1e-3)) < 1e-6 * d["value"]
