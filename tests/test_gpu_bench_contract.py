"""bench.py prints exactly one JSON line with the contract's keys (short run of the headline workload)."""
import json
import os
import subprocess
import sys

import pytest

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_one_json_line_with_roofline():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--steps", "3", "--warmup", "1", "--no-extras",
                        "--no-cpu"], stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=600)
    assert r.returncode == 0, r.stderr[-2000:]
    lines = [l for l in r.stdout.splitlines() if l.strip()]
    assert len(lines) == 1
    d = json.loads(lines[0])
    for k in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
              "vs_baseline", "dtype", "data", "config", "roofline"):
        assert k in d, k
    assert d["n_gpus"] == 1 and d["steps"] == 3 and d["vs_baseline"] is None and "workload" in d["config"]
    rf = d["roofline"]
    assert rf["bound"] == "hbm" and rf["peak"] == 8000 and abs(rf["frac"] - rf["achieved"] / rf["peak"]) < 1e-9
    assert 0.3 < rf["frac"] < 1.0 and d["value"] > 5e7
    assert 3000 < rf["copy_probe_gbs"] < rf["peak"]            # the measured plain-copy rate beside the nominal peak


def test_decode_figures_never_exceed_the_peak():
    """Every fraction the decode leg reports is a rate of bytes the timed launches really move: `frac` only for
    the kernels that run the reference's algorithm, `frac_of_bytes_moved` for the far-sum / windowed steps."""
    import torch
    sys.path.insert(0, ROOT)
    import bench
    d = bench.decode_layer_set(4096, torch.device("cuda:0"), 20, 3)
    assert "frac" not in d and d["us_per_step"] > 0 and d["reference_algorithm"]["us_per_step"] >= d["us_per_step"] * 0.9
    assert 0.2 < d["frac_reference_algorithm"] < 1.0 and 0.05 < d["frac_of_bytes_moved"] < 1.0
    for name, k in d["kernels"].items():
        fr = k.get("frac", k.get("frac_of_bytes_moved"))
        assert fr is not None and 0.0 < fr < 1.0, (name, k)
        assert ("frac" in k) != ("frac_of_bytes_moved" in k), name
    assert "frac_of_bytes_moved" in d["kernels"]["mr_step_far_sums"] and "frac" in d["kernels"]["mr_step_whole_cache"]
