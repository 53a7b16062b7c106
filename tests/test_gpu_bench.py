"""The benchmark's output contract, on a short run of the default workload."""

import json
import os
import subprocess
import sys

import pytest

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_bench_prints_one_json_line_with_the_agreed_fields():
    r = subprocess.run(
        [sys.executable, os.path.join(ROOT, "bench.py"), "--steps", "5", "--warmup", "2", "--settle-steps", "20",
         "--no-cpu-baseline"],
        capture_output=True, text=True, timeout=300, cwd=ROOT)
    assert r.returncode == 0, r.stderr[-2000:]
    lines = [ln for ln in r.stdout.splitlines() if ln.strip()]
    assert len(lines) == 1, r.stdout
    d = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better",
                "scaling", "vs_baseline", "dtype", "data", "config", "roofline"):
        assert key in d, key
    assert d["n_gpus"] == 1 and d["steps"] == 5 and d["warmup"] == 2 and d["unit"] == "tokens/s"
    assert d["vs_baseline"] is None and d["higher_is_better"] is True
    assert "workload" in d["config"] and "model" not in d["config"]
    roof = d["roofline"]
    for key in ("bound", "achieved", "peak", "unit", "frac", "traffic"):
        assert key in roof, key
    assert roof["bound"] == "hbm" and roof["unit"] == "GB/s" and roof["peak"] == 8000.0
    assert abs(roof["frac"] - roof["achieved"] / roof["peak"]) < 1e-9
    assert 0.2 < roof["frac"] < 1.0
    # tokens/s is B*T over the step time
    assert abs(d["value"] - 8 * 4096 / (d["ms_per_step"] * 1e-3)) < 1e-6 * d["value"]
    # the other configurations of the benchmark definition ride along as sub-records
    assert set(d["also"]) == {"scan_plain_alloc", "long", "scan_conv", "scan_gated", "gates", "block", "decode",
                              "model"}
    # the headline's tensors are placed as the library places its own; the same shape with plain
    # torch.empty rides along
    assert "activation_empty" in d["config"]["allocation"]
    assert d["also"]["scan_plain_alloc"]["config"]["allocation"].startswith("plain torch.empty")
    for name, rec in d["also"].items():
        assert rec["value"] > 0 and "workload" in rec["config"], name
        if name != "model":   # launch-bound end to end: no roofline is claimed for it
            assert 0.0 < rec["roofline"]["frac"] < 1.0, name
    for name in ("scan_plain_alloc", "long", "scan_conv", "scan_gated", "gates", "block"):
        assert d["also"][name]["roofline"]["frac"] > 0.2, name
    # a traffic figure is reported only when it was measured on the present kernel sources
    assert roof["traffic"] is None or roof["traffic"] > roof["algorithmic_bytes_per_launch"]
    assert (roof["traffic_frac"] is None) == (roof["traffic"] is None)
    assert roof["traffic_frac"] is None or roof["frac"] < roof["traffic_frac"] < 1.0
