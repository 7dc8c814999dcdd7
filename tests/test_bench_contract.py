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


def test_rows_of_the_printed_line_stay_short():
    """The driver keeps the last 8 KB of the output: the full default run prints the headline object (about 2 KB with
    the roofline, its nested prefill object and the CPU baseline) and 25 rows, which must fit with room to spare."""
    sys.path.insert(0, ROOT)
    import bench
    r = {"shape": "8x22b", "T": 8192, "logits": "two_experts", "mode": "f32_partials_f32out", "ms": 4.8123456789,
         "tokens_per_s": 1702345.678, "hbm_frac": 0.07712345, "mfma_frac": 0.4812345,
         "errors": {"max_abs": 0.00329732894, "mean_rel": 0.000213456789}, "meets_tolerance": False}
    row = json.dumps(bench.compact(r), separators=(",", ":"))
    e2e = json.dumps(bench.compact_e2e({"layers": 32, "requests": 100, "wall_s": 8.4123456, "output_tokens_per_s": 2136.123456,
                                        "prefill_tokens_per_s": 39876.54321, "decode_tokens_per_s": 2654.321,
                                        "moe_share_of_gpu_time": 0.5791234}), separators=(",", ":"))
    assert len(row) <= 200 and len(e2e) <= 200
    assert 25 * len(row) + len(e2e) + 2500 < 8000
    assert bench.sig(1716433.0658741253) == 1716000.0 and bench.sig(0.00021345678, 3) == 0.000213 and bench.sig(None) is None
    # the drop-in layer's form is the headline: w2 as float16, float32 output for the tolerance
    assert bench.MODES["default_f32out"] == bench.F_W2_F16 | bench.F_OUT_F32 and bench.MODES["default"] == bench.F_W2_F16


def test_routing_kinds_of_the_synthetic_batch():
    """`balanced` gives every expert exactly 2T/E rows (the tiled kernels' best case), `two_experts` sends every token
    to experts 0 and 1, `zipf` favours one expert; x is the same whatever the routing."""
    import torch
    sys.path.insert(0, ROOT)
    import bench
    dev, T = torch.device("cpu"), 256
    x0, lg = bench.make_batch(torch, dev, T, logits="normal")
    assert x0.shape == (T, bench.H) and lg.shape == (T, bench.E) and lg.dtype == torch.bfloat16
    counts = {}
    for kind in ("normal", "zipf", "two_experts", "balanced"):
        x, lg = bench.make_batch(torch, dev, T, logits=kind)
        assert torch.equal(x, x0)
        ids = lg.float().topk(bench.TOPK, dim=1).indices
        counts[kind] = torch.bincount(ids.flatten(), minlength=bench.E)
        assert int(counts[kind].sum()) == T * bench.TOPK
    assert counts["balanced"].tolist() == [T * bench.TOPK // bench.E] * bench.E
    assert counts["two_experts"].tolist() == [T, T] + [0] * (bench.E - 2)
    assert int(counts["zipf"].max()) > 2 * T * bench.TOPK // bench.E      # the busiest expert: more than twice its share
    assert int(counts["normal"].max()) < 2 * T * bench.TOPK // bench.E


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
    assert abs(r["frac"] - r["achieved"] / r["peak"]) < 1e-4            # both printed with five digits
    assert abs(r["achieved"] - r["per_launch"] / (r["avg_launch_ms"] * 1e-3) / 1e9) <= 1e-4 * r["achieved"]
    assert 0.5 < r["frac"] < 1.0
    assert d["config"]["mean_rel_err"] <= 1e-3 and d["config"]["max_abs_err"] <= 2e-2
    assert d["config"]["meets_tolerance_2e-2_1e-3"] is True and d["config"]["mode"] == "default_f32out"
    assert len(lines[0]) < 3000
    assert d["cpu_baseline"] is None      # --no-cpu
