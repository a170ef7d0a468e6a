"""The bench line the driver parses: one JSON object on stdout with the agreed keys, measured on the GPU."""
import json
import os
import subprocess
import sys

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.mark.gpu
def test_bench_prints_one_json_line_with_the_agreed_keys():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "1", "--steps", "5", "--warmup", "2",
                        "--no-extras", "--no-scaled", "--no-cpu-baseline"], capture_output=True, text=True, timeout=600)
    assert r.returncode == 0, r.stderr[-2000:]
    lines = [l for l in r.stdout.splitlines() if l.strip()]
    assert len(lines) == 1, lines
    out = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "roofline"):
        assert key in out, key
    assert out["n_gpus"] == 1 and out["steps"] == 5 and out["warmup"] == 2 and out["vs_baseline"] is None
    assert out["unit"] == "GB/s" and out["higher_is_better"] is True and "workload" in out["config"]
    roof = out["roofline"]
    assert roof["bound"] == "hbm" and roof["peak"] == 8000.0 and roof["unit"] == "GB/s"
    assert abs(roof["frac"] - roof["achieved"] / roof["peak"]) < 1e-3
    assert 500.0 < out["value"] < 8000.0 and 0.05 < roof["frac"] < 1.0
    # bytes of one step over its time is the value
    assert abs(out["value"] - 2 * roof["algorithmic_bytes"] / (out["ms_per_step"] * 1e-3) / 1e9) < 0.01 * out["value"]
    assert roof["traffic"] is None or roof["traffic"] >= roof["algorithmic_bytes"]


def test_bench_refuses_more_than_one_gpu():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert r.returncode != 0 and "ONE GPU" in (r.stderr + r.stdout)
