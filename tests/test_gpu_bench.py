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


def test_stream_probe_moves_all_of_every_tensor():
    """hawk_stream_probe: every 32-bit word of output i is the sum of the inputs' words at its place
    plus i, flat, tiled in memory order and tiled in the scan's launch order (sequences of 2 row
    groups: position along the sequence slowest), for every supported mix; other mixes and shapes are
    refused."""
    import ctypes

    import torch
    from hawk_pytorch_amd import _lib

    lib = _lib.load()
    rows, pitch = 512, 1280          # four row groups of 128 rows; bytes per row: five column tiles of 256 bytes
    n = rows * pitch // 4
    gen = torch.Generator(device="cuda").manual_seed(4)
    ins = [torch.randint(0, 1 << 20, (n,), dtype=torch.int32, device="cuda", generator=gen) for _ in range(5)]
    st = torch.cuda.current_stream().cuda_stream
    for nr, nw in ((1, 1), (1, 2), (1, 3), (2, 1), (3, 1), (5, 3)):
        for shape in (0, 1, 2):
            if shape == 0 and (n * 4) % 16384:
                continue
            outs = [torch.full((n,), -1, dtype=torch.int32, device="cuda") for _ in range(nw)]
            r = (ctypes.c_void_p * nr)(*[t.data_ptr() for t in ins[:nr]])
            w = (ctypes.c_void_p * nw)(*[t.data_ptr() for t in outs])
            _lib.check("hawk_stream_probe", lib.hawk_stream_probe(r, nr, w, nw, n * 4, pitch, shape, st))
            torch.cuda.synchronize()
            want = sum(ins[:nr])
            for i, o in enumerate(outs):
                assert torch.equal(o, want + i), (nr, nw, shape, i)
    r = (ctypes.c_void_p * 2)(ins[0].data_ptr(), ins[1].data_ptr())
    w = (ctypes.c_void_p * 2)(ins[2].data_ptr(), ins[3].data_ptr())
    assert lib.hawk_stream_probe(r, 2, w, 2, n * 4, pitch, 0, st) == _lib.HAWK_ERR_BAD_SHAPE      # no 2 + 2
    assert lib.hawk_stream_probe(r, 2, w, 1, n * 4, pitch + 4, 1, st) == _lib.HAWK_ERR_BAD_SHAPE  # pitch % 256
    assert lib.hawk_stream_probe(r, 2, w, 1, n * 4 - 16384, pitch, 1, st) == _lib.HAWK_ERR_BAD_SHAPE
    assert lib.hawk_stream_probe(r, 2, w, 1, n * 4, pitch, 3, st) == _lib.HAWK_ERR_BAD_SHAPE      # 4 groups % 3
    assert lib.hawk_stream_probe(r, 2, w, 1, n * 4, pitch, -1, st) == _lib.HAWK_ERR_BAD_SHAPE
