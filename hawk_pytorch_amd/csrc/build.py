"""Builds libhawk_hip.so (the C-ABI HIP library) in-tree with hipcc for gfx950.

Usage:  python -m hawk_pytorch_amd.csrc.build [--force]
"""

from __future__ import annotations

import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

CSRC = os.path.dirname(os.path.abspath(__file__))
LIB_NAME = "libhawk_hip.so"
LIB_PATH = os.path.join(CSRC, LIB_NAME)
SOURCES = ["hawk_scan.hip", "hawk_conv.hip", "hawk_step.hip", "hawk_gates.hip", "hawk_block.hip", "hawk_probe.hip", "hawk_capi.hip"]
HEADERS = ["hawk_scan.h", "hawk_device.h", "hawk_reduce.h", os.path.join("..", "..", "include", "hawk_hip.h")]

# Packed-FP32 VALU instructions are switched off for all device code.
HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall",
    "-Wno-unused-function",
]


def _hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; libhawk_hip.so cannot be built")
    return exe


def _run(cmd):
    proc = subprocess.run(cmd, cwd=CSRC, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError("command failed: %s\n%s\n%s" % (" ".join(cmd), proc.stdout, proc.stderr))
    return proc


def build(force: bool = True, verbose: bool = False) -> str:
    """Compile every translation unit and link the shared library.  Returns its path."""
    hipcc = _hipcc()
    objdir = os.path.join(CSRC, "build")
    os.makedirs(objdir, exist_ok=True)
    newest_header = max(os.path.getmtime(os.path.join(CSRC, h)) for h in HEADERS)

    def compile_one(src):
        obj = os.path.join(objdir, src.replace(".hip", ".o"))
        src_path = os.path.join(CSRC, src)
        stale = (
            force
            or not os.path.exists(obj)
            or os.path.getmtime(obj) < max(os.path.getmtime(src_path), newest_header)
        )
        if stale:
            if verbose:
                print("hipcc", src, flush=True)
            _run([hipcc, *HIPCC_FLAGS, "-c", src_path, "-o", obj])
        return obj

    with ThreadPoolExecutor(max_workers=len(SOURCES)) as pool:
        objs = list(pool.map(compile_one, SOURCES))
    _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB_PATH, *objs])
    return LIB_PATH


if __name__ == "__main__":
    path = build(force="--force" in sys.argv, verbose=True)
    print(path)
