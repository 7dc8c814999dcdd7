"""bench.py's contract: the one-GPU refusal and the figures its roofline is quoted on (host side), and the JSON line of
a short run on the GPU."""
import json
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BENCH = os.path.join(ROOT, "bench.py")


def test_more_than_one_gpu_is_refused_with_a_message():
    p = subprocess.run([sys.executable, BENCH, "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert p.returncode != 0
    assert "one GPU" in p.stderr or "--gpus 1" in p.stderr
    assert p.stdout.strip() == ""


def test_algorithmic_work_of_the_layer():
    sys.path.insert(0, ROOT)
    import bench
    H, I = 4096, 14336
    assert (bench.H, bench.I, bench.E, bench.TOPK) == (H, I, 8, 2)
    # all eight experts active: every weight byte once, plus x, out (fp32 out is counted as bf16 rows) and the logits
    weights = 8 * 3 * H * I * 2
    assert weights <= bench.layer_bytes(64, 8) <= weights + 64 * H * 8 + 64 * 8 * 4
    assert bench.layer_bytes(1, 2) < bench.layer_bytes(1, 8)
    assert bench.layer_flops(8192) == 8192 * 2 * 6 * H * I


@pytest.mark.gpu
def test_json_line_of_a_short_run():
    p = subprocess.run([sys.executable, BENCH, "--steps", "5", "--warmup", "2", "--no-table", "--no-cpu"],
                       capture_output=True, text=True, timeout=300, cwd=ROOT)
    assert p.returncode == 0, p.stderr[-2000:]
    lines = [l for l in p.stdout.splitlines() if l.strip()]
    assert len(lines) == 1
    d = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline"):
        assert key in d, key
    assert d["n_gpus"] == 1 and d["steps"] == 5 and d["warmup"] == 2 and d["vs_baseline"] is None
    assert d["unit"] == "tokens/s" and d["higher_is_better"] is True and d["data"] == "synthetic"
    assert "workload" in d["config"] and "model" not in d["config"]
    assert abs(d["value"] - 64 / (d["ms_per_step"] * 1e-3)) <= 1e-6 * d["value"]
    r = d["roofline"]
    assert r["bound"] == "hbm" and r["peak"] == 8000.0 and r["unit"] == "GB/s"
    assert abs(r["frac"] - r["achieved"] / r["peak"]) < 1e-9
    assert abs(r["achieved"] - r["per_launch"] / (r["avg_launch_ms"] * 1e-3) / 1e9) <= 1e-6 * r["achieved"]
    assert 0.5 < r["frac"] < 1.0
    assert d["config"]["errors_vs_fp32_oracle"]["mean_rel"] <= 1e-3
    assert d["cpu_baseline"] is None      # --no-cpu
