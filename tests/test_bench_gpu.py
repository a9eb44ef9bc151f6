"""bench.py's output contract: one JSON line with the agreed keys, a roofline object whose figures are consistent with each other,
and a refusal of more than one GPU."""
import json
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_bench_refuses_more_than_one_gpu():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=300)
    assert r.returncode != 0
    assert "one GPU" in r.stdout


@pytest.mark.gpu
@pytest.mark.parametrize("workload,instances", [("resnet18", 1), ("yolov3_tiny", 2)])
def test_bench_prints_one_json_line_with_the_contract_keys(workload, instances):
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--workload", workload, "--steps", "24", "--warmup", "6", "--instances", str(instances),
                        "--no-cpu-baseline"], stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=600, cwd=ROOT)
    assert r.returncode == 0, r.stderr[-2000:]
    lines = [l for l in r.stdout.splitlines() if l.strip()]
    assert len(lines) == 1, lines
    d = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling", "vs_baseline", "dtype", "data", "config",
                "roofline"):
        assert key in d, key
    assert d["n_gpus"] == 1 and d["steps"] == 24 and d["warmup"] == 6 and d["higher_is_better"] is True and d["vs_baseline"] is None
    assert d["unit"] == "images/s" and d["data"] == "synthetic" and d["dtype"] in ("f16", "f32")
    assert "workload" in d["config"] and workload.split("_")[0] in d["config"]["workload"] and "model" not in d["config"]
    assert d["config"]["instances"] == instances
    assert d["value"] > 0 and d["ms_per_step"] > 0
    rf = d["roofline"]
    for key in ("bound", "achieved", "peak", "unit", "frac", "traffic"):
        assert key in rf, key
    assert rf["bound"] in ("hbm", "mfma") and rf["unit"] in ("GB/s", "TFLOP/s")
    assert 0 < rf["achieved"] < rf["peak"]
    assert abs(rf["frac"] - rf["achieved"] / rf["peak"]) < 2e-4
    # achieved = FLOPs of one pass over the convolution launches / their summed duration
    assert abs(rf["achieved"] - rf["flops_per_step"] / (rf["launches_per_step"] * rf["avg_launch_us"] * 1e-6) / 1e12) <= 0.01 * rf["achieved"]
    # the attainable bound: every convolution launch against max(FLOPs / MFMA peak, least bytes / HBM peak), split by the binding roof
    assert 0 < rf["attainable_frac"] <= 1.0 and len(rf["plan_hash"]) == 16
    split = rf["by_binding_roof"]
    n = split["mfma_bound"]["launches"] + split["hbm_bound"]["launches"]
    assert n >= rf["launches_per_step"] - 1 and n <= rf["launches_per_step"] + 2          # (+ the connected layer where it is not lowered to a convolution)
    t = split["mfma_bound"]["us"] + split["hbm_bound"]["us"]
    t_min = split["mfma_bound"]["us_min"] + split["hbm_bound"]["us_min"]
    assert abs(rf["attainable_frac"] - t_min / t) < 5e-3
    for c in ("mfma_bound", "hbm_bound"):
        assert split[c]["us_min"] <= split[c]["us"]
    assert rf["traffic"] is None or rf["traffic"] > 0
