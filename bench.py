#!/usr/bin/env python3
"""Benchmark of the RG-LRU scan hot path on one MI355X.

A step is one forward scan plus one backward scan over one synthetic batch, called
through the C ABI of libhawk_hip.so with every buffer already resident in HBM and
pre-allocated (nothing is allocated inside the timed region).

Default workload: B=8, T=4096, D=2560, bf16 activations, fp32 state (the configuration
the 70 %-of-HBM-peak target is quoted on).  ``--workload long`` runs B=2, T=32768,
D=4096; ``--workload scan_conv`` adds the temporal conv1d forward and backward;
``--workload scan_gated`` runs the scan fused with the block's gate (out = gelu(y) * h,
y being one half of a [B, T, 2D] projection), 12 + 20 bytes per element;
``--workload gates`` runs the fused block-diagonal gate projections (matrix-core kernels:
forward, input gradient, weight gradients) on 32768 tokens, D = 2560, 10 blocks, bf16;
``--workload block`` chains the whole recurrent core of one layer at B=8, T=4096, D=2560 (conv and
both gate projections in one kernel, scan fused with the output gate, and the backward of all of
them) through the C ABI on the [B,T,2D] output of the block's input projection in place, one host call
per direction: six large launches that move 30 activation-sized tensors, one that rounds the fp32
weights of both gates to bf16 (as the Python host does at this size) and one for the three closing
reductions of the backward; ``--unfused-conv`` runs the single entry points instead (the conv as a
launch of its own on a copy of the x half, seven large launches and 31 tensors, two weight casts,
a reduction launch per backward call);
``--workload model`` runs full training steps (forward, backward, AdamW) of the upstream
README model (vocabulary 32000, hidden = recurrent = 512, MLP 1024, 8 layers, 16 gate blocks)
on a 1 x 2048 batch under bf16 autocast, with and without the fused gate / epilogue kernels;
``--workload decode`` times one-token steps of a 26-layer Hawk (R = H = 2560, I = 7680,
10 gate blocks, vocabulary 32000, bf16 weights) at batch 256 after a 1024-token prefill,
eagerly and as a replayed HIP graph, plus the one-launch recurrent core of a layer and token
(hawk_decode_core_step_ws, the kernel the model launches) on its own.

Timing.  The timed region of the kernel workloads holds nothing but the launches, between one
event and one host clock reading on either side: `ms_per_step` and `value` come from it.  An
event recorded between two launches makes the next dispatch wait behind a marker packet, 3-4 us
each on this GPU, which no training loop pays; the per-launch durations that the `roofline`
and `fwd` figures divide by are therefore measured on the same steps run once more, right behind
the timed region, with a HIP event after every launch (`launch_timing_region`).
`stream_ceiling` (default workload) times stock PyTorch streaming kernels with the forward's and
the backward's read/write mix on the same tensors in the same process.

The kernel workloads (scan*, long, gates, block) run ``--settle-steps`` untimed steps (default 100)
before the ``--warmup`` ones: for about 50 steps (20 ms) after the GPU leaves idle the same kernels
run up to 12 % slower than they do from then on.

The default workload's line also carries, under "also", records for the long-context, the
scan + conv and the gated-scan configurations, the gate projections, the recurrent core of one
layer, the decode step and the README model's training step, timed after the headline region in the same process with a quarter of the steps
(``--no-also`` leaves them out).

Prints one JSON line:
  value        tokens/s = B*T / (wall time per step), whole job on one GPU
  roofline     for the dominant kernel (the backward scan): algorithmic bytes per launch
               (16 B/element in bf16: five tensors read, three written) over the mean
               duration of the backward launch measured with HIP events on the launch
               stream, against the 8 TB/s HBM peak; `traffic` is the launch's HBM bytes as
               rocprofv3 counted them (profiles/hbm_traffic.json, while its digest matches the
               kernel sources) and `traffic_frac` the same launch time against those bytes
  cpu_baseline the PyTorch CPU loop over time of the same recurrence (forward + autograd
               backward, fp32) on this host's cores, on a bounded sample of the workload
"""

from __future__ import annotations

import argparse
import ctypes
import json
import os
import sys
import time

import numpy as np
import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0

# HBM bytes per launch of each workload's dominant kernel, as rocprofv3 counted them
# (--pmc FETCH_SIZE, then WRITE_SIZE, each scaled by what the same counter reads for a plain
# device copy of known size in the same run), are kept in profiles/hbm_traffic.json together
# with the digest of the kernel sources they were measured on.  A record taken on other
# sources is stale and is not reported.
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "hbm_traffic.json")
KERNEL_SOURCES = {"gates": ("hawk_gates.hip", "hawk_device.h", "hawk_reduce.h"),
                  "scan_conv": ("hawk_scan.hip", "hawk_conv.hip", "hawk_device.h", "hawk_reduce.h")}
SCAN_KERNEL_SOURCES = ("hawk_scan.hip", "hawk_device.h", "hawk_reduce.h")


def kernel_source_digest(workload):
    """Digest of the sources of the kernels that `workload` times."""
    import hashlib

    h = hashlib.sha256()
    for name in KERNEL_SOURCES.get(workload, SCAN_KERNEL_SOURCES):
        with open(os.path.join(ROOT, "hawk_pytorch_amd", "csrc", name), "rb") as f:
            h.update(f.read())
    return h.hexdigest()[:16]


def measured_traffic(workload):
    """FETCH + WRITE bytes per launch recorded for `workload`, or None (no record, or a record
    taken on kernel sources other than the present ones)."""
    try:
        with open(TRAFFIC_FILE) as f:
            rec = json.load(f).get(workload)
    except (OSError, ValueError):
        return None
    if not rec or rec.get("kernel_source_digest") != kernel_source_digest(workload):
        return None
    return float(rec["fetch_bytes"]) + float(rec["write_bytes"])


def record_traffic(workload, fetch_bytes, write_bytes, note):
    """Write one record of profiles/hbm_traffic.json (used after a rocprofv3 --pmc pass)."""
    import datetime
    import subprocess

    try:
        with open(TRAFFIC_FILE) as f:
            data = json.load(f)
    except (OSError, ValueError):
        data = {}
    try:
        commit = subprocess.run(["git", "-C", ROOT, "rev-parse", "--short", "HEAD"], capture_output=True,
                                text=True).stdout.strip() or None
    except OSError:
        commit = None
    data[workload] = {
        "fetch_bytes": float(fetch_bytes), "write_bytes": float(write_bytes),
        "kernel_source_digest": kernel_source_digest(workload), "commit_before": commit,
        "date": datetime.date.today().isoformat(), "note": note,
    }
    with open(TRAFFIC_FILE, "w") as f:
        json.dump(data, f, indent=1, sort_keys=True)
        f.write("\n")


WORKLOADS = {
    # name: (B, T, D, a^8 range, includes conv)
    "scan": (8, 4096, 2560, (0.9, 0.999), False),
    "long": (2, 32768, 4096, (0.99, 0.9999), False),
    "scan_conv": (8, 4096, 2560, (0.9, 0.999), True),
    "scan_gated": (8, 4096, 2560, (0.9, 0.999), False),
    # fp32 activations and gate logits in, bf16 h and grad_out, fp32 gradients out (what the
    # scan sees under bf16 autocast when its producers ran in fp32)
    "scan_mixed": (8, 4096, 2560, (0.9, 0.999), False),
}


def lambda_for_a8_range(gen, D, lo, hi):
    u = torch.empty(D, dtype=torch.float64).uniform_(lo, hi, generator=gen)
    return torch.log(u.pow(-1.0 / 8.0) - 1.0).float()


def cpu_baseline(B, D, lo, hi, seed, budget_elements=1024 * 8 * 2560):
    """The recurrence on this host's cores, on the first time rows of the workload's shape
    (about `budget_elements` element-steps), forward plus backward in fp32, two ways:

    * `value`: the PyTorch loop over time (oracle/rglru_torch.py: the one-token step of
      hawk/hawk.py:137-151, :196 iterated, autograd for the backward), 10-20 s on 16 host
      threads.  Its rate falls with the sample's length, because the autograd tape grows.
    * `scalar_c`: the single-threaded C restatement of the two kernels' arithmetic
      (oracle_rglru_scan_{fwd,bwd}_f32, following hawk/scan_fused.py:44-109 and :123-317), whose
      rate does not depend on the length of the sample.
    """
    import oracle
    from oracle import rglru_torch

    gen = torch.Generator().manual_seed(seed)
    T = max(256, budget_elements // (B * D))
    x, xg, ag, go = (torch.randn(B, T, D, generator=gen) for _ in range(4))
    lam = lambda_for_a8_range(gen, D, lo, hi)
    rglru_torch.rglru_scan_fwd_bwd(x[:, :8], xg[:, :8], ag[:, :8], lam, go[:, :8])  # warm-up
    t0 = time.perf_counter()
    rglru_torch.rglru_scan_fwd_bwd(x, xg, ag, lam, go)
    dt = time.perf_counter() - t0

    xn, xgn, agn, gon, lamn = (t.numpy() for t in (x, xg, ag, go, lam))
    oracle.rglru_scan_fwd(xn[:, :8], xgn[:, :8], agn[:, :8], lamn, precision="f32")  # loads the library
    t0 = time.perf_counter()
    hn = oracle.rglru_scan_fwd(xn, xgn, agn, lamn, precision="f32")
    oracle.rglru_scan_bwd(xn, xgn, agn, lamn, hn, gon, precision="f32")
    dt_c = time.perf_counter() - t0
    return {
        "value": B * T / dt,
        "unit": "tokens/s",
        "cores": torch.get_num_threads(),
        "kind": "port",
        "sample": f"first {T} of the time rows at B={B}, D={D}, fp32, forward + autograd backward, "
                  f"{dt:.2f} s, host has {os.cpu_count()} logical cpus",
        "scalar_c": {
            "value": B * T / dt_c, "unit": "tokens/s", "cores": 1, "kind": "port",
            "sample": f"the same {T} rows through the scalar C port of both kernels, fp32, {dt_c:.2f} s",
        },
    }


ALLOCATION = {
    False: "every tensor placed as the library's host code places the activations it allocates: base addresses "
           "256 bytes apart modulo 1 KiB (hawk_pytorch_amd._lib.activation_empty); --plain-alloc for torch.empty",
    True: "plain torch.empty (large blocks start on 2 MiB boundaries)",
}


def act_empty(args, shape, dtype, dev):
    """An activation tensor placed as the library's host code places the ones it allocates (base
    addresses 256 bytes apart modulo 1 KiB, hawk_pytorch_amd._lib.activation_empty), or by a
    plain torch.empty with --plain-alloc."""
    from hawk_pytorch_amd import _lib

    if args.plain_alloc:
        return torch.empty(shape, dtype=dtype, device=dev)
    return _lib.activation_empty(shape, dtype, dev)


def act_randn(args, shape, dtype, dev, gen):
    t = act_empty(args, shape, dtype, dev)
    t.copy_(torch.randn(shape, device=dev, generator=gen).to(dtype))
    return t


def run_gates(args, lib, dev):
    """Both gate projections of a layer on B*T = 32768 tokens: forward, dx, dw/db."""
    from hawk_pytorch_amd import _lib

    M, D, nb = 8 * 4096, 2560, 10
    bw = D // nb
    bf, code, f32 = torch.bfloat16, _lib.HAWK_DTYPE_BF16, _lib.HAWK_DTYPE_F32
    gen = torch.Generator(device=dev).manual_seed(args.seed)
    x, gi, ga = (act_randn(args, (M, D), bf, dev, gen) for _ in range(3))
    wi, wa = (torch.randn(nb, bw, bw, device=dev, generator=gen) / bw ** 0.5 for _ in range(2))
    bi, ba = (torch.randn(D, device=dev, generator=gen) for _ in range(2))
    oi, oa, dx = (act_empty(args, (M, D), bf, dev) for _ in range(3))
    dwi, dwa = torch.empty_like(wi), torch.empty_like(wa)
    dbi, dba = torch.empty_like(bi), torch.empty_like(ba)
    nws = lib.hawk_gate_proj_bwd_weights_workspace_bytes(M, D, nb)
    ws = torch.empty(nws, dtype=torch.uint8, device=dev)
    stream = torch.cuda.current_stream(dev).cuda_stream

    # As the Python host does from 8192 rows on, the fp32 weights are rounded to bf16 once per step
    # (two small kernels, inside the step but outside the three brackets) instead of by every
    # workgroup of both kernels that read them; --fp32-gate-weights hands the kernels the fp32 ones.
    wi16, wa16 = torch.empty_like(wi, dtype=bf), torch.empty_like(wa, dtype=bf)
    cast = not args.fp32_gate_weights
    kwi, kwa, wcode = (wi16, wa16, code) if cast else (wi, wa, f32)

    def round_weights():
        if cast:
            wi16.copy_(wi)
            wa16.copy_(wa)

    def fwd():
        _lib.check("gate_proj_fwd", lib.hawk_gate_proj_fwd(
            x.data_ptr(), kwi.data_ptr(), bi.data_ptr(), kwa.data_ptr(), ba.data_ptr(), oi.data_ptr(), oa.data_ptr(),
            M, D, nb, code, wcode, code, stream))

    def bwd_input():
        _lib.check("gate_proj_bwd_input", lib.hawk_gate_proj_bwd_input(
            gi.data_ptr(), ga.data_ptr(), kwi.data_ptr(), kwa.data_ptr(), None, dx.data_ptr(), M, D, nb, code, wcode,
            code, stream))

    def bwd_weights():
        _lib.check("gate_proj_bwd_weights", lib.hawk_gate_proj_bwd_weights(
            x.data_ptr(), gi.data_ptr(), ga.data_ptr(), dwi.data_ptr(), dbi.data_ptr(), dwa.data_ptr(),
            dba.data_ptr(), M, D, nb, code, code, ws.data_ptr(), nws, stream))

    if args.calibration_copy:
        for _ in range(3):
            oi.copy_(x)
        torch.cuda.synchronize()
    for _ in range(args.settle_steps + args.warmup):
        round_weights(), fwd(), bwd_input(), bwd_weights()
    torch.cuda.synchronize()
    # timed region: the launches alone (an event between two launches costs the GPU 3-4 us)
    t0 = time.perf_counter()
    for k in range(args.steps):
        round_weights(), fwd(), bwd_input(), bwd_weights()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    ms_per_step = wall * 1e3 / args.steps
    # launch durations: the same steps again with an event after every launch
    ev = [[torch.cuda.Event(enable_timing=True) for _ in range(4)] for _ in range(args.steps)]
    for k in range(args.steps):
        round_weights()
        ev[k][0].record()
        fwd()
        ev[k][1].record()
        bwd_input()
        ev[k][2].record()
        bwd_weights()
        ev[k][3].record()
    torch.cuda.synchronize()
    ms = [float(np.mean([e[i].elapsed_time(e[i + 1]) for e in ev])) for i in range(3)]
    N = M * D
    # forward: read x, write two logits; dx: read two gradients, write dx; dw: read x and two gradients
    alg = [3 * 2 * N, 3 * 2 * N, 3 * 2 * N]
    flops = [4.0 * N * bw] * 3
    gbs = [alg[i] / (ms[i] * 1e-3) / 1e9 for i in range(3)]
    out = {
        "metric": "fused gate projections fwd+bwd tokens/s, 1 GPU",
        "value": M / (ms_per_step * 1e-3),
        "unit": "tokens/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "settle_steps": args.settle_steps,
        "ms_per_step": ms_per_step,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16 operands, f32 accumulation",
        "data": f"synthetic, seed {args.seed}: activations and gradients ~ N(0,1), weights ~ N(0, 1/bw)",
        "config": {"workload": f"gates: both block-diagonal gate projections fwd + input grad + weight grads, "
                               f"M={M}, D={D}, {nb} blocks of {bw}, bf16, fp32 weights "
                               + ("rounded to bf16 once per step" if cast else "rounded by every workgroup"),
                   "M": M, "D": D, "num_blocks": nb, "allocation": ALLOCATION[bool(args.plain_alloc)]},
        "roofline": {
            "bound": "hbm",
            "kernel": "gate_proj_bwd_weights_kernel (+ gate_proj_reduce_kernel, same launch call)",
            "achieved": gbs[2], "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": gbs[2] / HBM_PEAK_GBS,
            "traffic": measured_traffic("gates"),
            "algorithmic_bytes_per_launch": alg[2], "launch_ms": ms[2],
        },
        "kernels": {name: {"ms": ms[i], "GBs": gbs[i], "frac": gbs[i] / HBM_PEAK_GBS,
                           "TFLOPs": flops[i] / (ms[i] * 1e-3) / 1e12}
                    for i, name in enumerate(("fwd", "bwd_input", "bwd_weights"))},
    }
    return out


def run_block(args, lib, dev):
    """conv -> gate projections -> gated scan, forward and backward, bf16 end to end."""
    from hawk_pytorch_amd import _lib

    B, T, D, nb, W = 8, 4096, 2560, 10, 4
    M, bw, N = B * T, D // nb, B * T * D
    bf, code = torch.bfloat16, _lib.HAWK_DTYPE_BF16
    gen = torch.Generator(device=dev).manual_seed(args.seed)
    xy = act_randn(args, (B, T, 2 * D), bf, dev, gen)
    xin = xy[..., :D].contiguous()          # conv input; the gate half stays in place
    y = xy[..., D:]
    gout = act_randn(args, (B, T, D), bf, dev, gen)
    cw = (torch.randn(W, D, device=dev, generator=gen) * 0.5).float()
    cb = torch.zeros(D, device=dev)
    wi, wa = (torch.randn(nb, bw, bw, device=dev, generator=gen) / bw ** 0.5 for _ in range(2))
    bi, ba = (torch.randn(D, device=dev, generator=gen) * 0.1 for _ in range(2))
    lam = lambda_for_a8_range(torch.Generator().manual_seed(args.seed), D, 0.9, 0.999).to(dev)
    e = lambda: act_empty(args, (B, T, D), bf, dev)  # noqa: E731
    u, xg, ag, h, out = e(), e(), e(), e(), e()
    du, dxg, dag, dy, dxin = e(), e(), e(), e(), e()
    dxy = act_empty(args, (B, T, 2 * D), bf, dev)   # gradient of xy, both halves written in place
    dlam = torch.empty(D, device=dev)
    dwi, dwa, dbi, dba = torch.empty_like(wi), torch.empty_like(wa), torch.empty_like(bi), torch.empty_like(ba)
    dcw, dcb = torch.empty_like(cw), torch.empty_like(cb)
    ws = torch.zeros(lib.hawk_scan_workspace_bytes(B, T, D, code), dtype=torch.uint8, device=dev)
    gws = torch.empty(lib.hawk_gate_proj_bwd_weights_workspace_bytes(M, D, nb), dtype=torch.uint8, device=dev)
    cws = torch.empty(lib.hawk_conv1d_bwd_workspace_bytes(B, T, D, W), dtype=torch.uint8, device=dev)
    st = torch.cuda.current_stream(dev).cuda_stream
    p = lambda t: t.data_ptr()  # noqa: E731

    w16 = torch.empty((2, nb, bw, bw), device=dev, dtype=bf)
    wi16, wa16 = w16[0], w16[1]
    F32 = _lib.HAWK_DTYPE_F32

    def fwd():
        if not args.unfused_conv:
            # one host call: the fp32 gate weights rounded to bf16 once per step (one launch for both
            # gates, inside the timed region), conv and both projections in one kernel reading the x
            # half of xy in place, then the scan with the output gate
            _lib.check("block_core_fwd", lib.hawk_block_core_fwd(
                p(xy), 2 * D, p(cw), p(cb), p(wi), p(bi), p(wa), p(ba), F32, p(w16), p(lam), p(u), p(xg), p(ag),
                p(h), p(out), None, B, T, D, nb, W, p(ws), ws.numel(), st))
            return
        # the single calls, as the Python host does from 8192 rows on: the fp32 gate weights are
        # rounded to bf16 once per step instead of by every workgroup
        wi16.copy_(wi)
        wa16.copy_(wa)
        _lib.check("conv_fwd", lib.hawk_conv1d_fwd(p(xin), p(cw), p(cb), None, p(u), B, T, D, W, code, code, st))
        _lib.check("gate_fwd", lib.hawk_gate_proj_fwd(p(u), p(wi16), p(bi), p(wa16), p(ba), p(xg), p(ag), M, D,
                                                      nb, code, code, code, st))
        _lib.check("scan_gated_fwd", lib.hawk_rglru_scan_gated_fwd(
            p(u), p(xg), p(ag), p(lam), p(y), 2 * D, p(h), p(out), None, B, T, D, code, code, p(ws), ws.numel(), st))

    def bwd():
        if not args.unfused_conv:
            # one host call: gated scan -> the projections' input gradient onto the scan's, in place
            # -> conv (right behind the kernel that wrote its input gradient: part of those 168 MB is
            # then still in the memory-side cache, 1 % of the step) -> the projections' weight
            # gradients -> one launch for the three closing reductions
            _lib.check("block_core_bwd", lib.hawk_block_core_bwd(
                p(xy), 2 * D, p(u), p(xg), p(ag), p(h), p(cw), p(wi16), p(wa16), code, p(lam), p(gout), p(dxy),
                2 * D, p(du), p(dxg), p(dag), p(dcw), p(dcb), p(dwi), p(dbi), p(dwa), p(dba), p(dlam), B, T, D, nb,
                W, p(ws), ws.numel(), p(gws), gws.numel(), p(cws), cws.numel(), st))
            return
        _lib.check("scan_gated_bwd", lib.hawk_rglru_scan_gated_bwd(
            p(u), p(xg), p(ag), p(lam), p(y), 2 * D, p(h), p(gout), p(du), p(dxg), p(dag), p(dy), D, p(dlam),
            B, T, D, code, code, p(ws), ws.numel(), st))
        _lib.check("gate_bwd_input", lib.hawk_gate_proj_bwd_input(p(dxg), p(dag), p(wi16), p(wa16), p(du), p(du), M,
                                                                  D, nb, code, code, code, st))
        _lib.check("conv_bwd", lib.hawk_conv1d_bwd(p(du), p(xin), p(cw), p(dxin), p(dcw), p(dcb), B, T, D, W,
                                                   code, code, p(cws), cws.numel(), st))
        _lib.check("gate_bwd_weights", lib.hawk_gate_proj_bwd_weights(
            p(u), p(dxg), p(dag), p(dwi), p(dbi), p(dwa), p(dba), M, D, nb, code, code, p(gws), gws.numel(), st))

    for _ in range(args.settle_steps + args.warmup):
        fwd(), bwd()
    torch.cuda.synchronize()
    # timed region: the launches alone (an event between two launches costs the GPU 3-4 us)
    t0 = time.perf_counter()
    for k in range(args.steps):
        fwd(), bwd()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    # forward / backward split: the same steps again with events around both halves
    ev = [[torch.cuda.Event(enable_timing=True) for _ in range(3)] for _ in range(args.steps)]
    for k in range(args.steps):
        ev[k][0].record()
        fwd()
        ev[k][1].record()
        bwd()
        ev[k][2].record()
    torch.cuda.synchronize()
    flag = ctypes.c_int(0)
    _lib.check("status", lib.hawk_scan_workspace_status(ws.data_ptr(), st, ctypes.byref(flag)))
    assert flag.value == 0 and bool(torch.isfinite((dxin if args.unfused_conv else dxy).float()).all())
    fwd_ms = float(np.mean([e_[0].elapsed_time(e_[1]) for e_ in ev]))
    bwd_ms = float(np.mean([e_[1].elapsed_time(e_[2]) for e_ in ev]))
    ms_per_step = wall * 1e3 / args.steps
    # tensors moved: conv 2, gates 3 (conv + gates in one kernel: 4), gated scan 6 | gated scan 10,
    # gate dx 4, gate dw 3, conv 3
    fwd_bytes, bwd_bytes = (11 if args.unfused_conv else 10) * 2 * N, 20 * 2 * N
    step_gbs = (fwd_bytes + bwd_bytes) / (ms_per_step * 1e-3) / 1e9
    return {
        "metric": "Hawk recurrent core (conv, gate projections, gated scan) fwd+bwd tokens/s, 1 GPU",
        "value": B * T / (ms_per_step * 1e-3), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "settle_steps": args.settle_steps, "ms_per_step": ms_per_step,
        "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16 activations, f32 parameters, state and accumulation",
        "data": f"synthetic, seed {args.seed}",
        "config": {"workload": f"block: conv1d(4) + gate projections ({nb} blocks) + scan fused with gelu(y)*h, "
                               f"fwd+bwd, B={B}, T={T}, D={D}, bf16", "B": B, "T": T, "D": D,
                   "allocation": ALLOCATION[bool(args.plain_alloc)]},
        "roofline": {"bound": "hbm", "kernel": "all launches of the step", "achieved": step_gbs,
                     "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": step_gbs / HBM_PEAK_GBS, "traffic": None,
                     "algorithmic_bytes_per_launch": fwd_bytes + bwd_bytes},
        "fwd": {"ms": fwd_ms, "GBs": fwd_bytes / (fwd_ms * 1e-3) / 1e9},
        "bwd": {"ms": bwd_ms, "GBs": bwd_bytes / (bwd_ms * 1e-3) / 1e9},
    }


def run_model(args, lib, dev):
    """Training steps of the README model at batch 1 x 2048, bf16 autocast."""
    import hawk_pytorch_amd as hk

    B, T, vocab = 1, 2048, 32000
    gen = torch.Generator(device=dev).manual_seed(args.seed)
    ids = torch.randint(1, vocab, (B, T), device=dev, generator=gen)

    def time_steps(**flags):
        torch.manual_seed(args.seed)
        cfg = hk.HawkConfig(vocab_size=vocab, hidden_size=512, intermediate_size=1024, num_hidden_layers=8,
                            recurrent_size=512, num_blocks=16, conv_width=4, **flags)
        with torch.device(dev):
            model = hk.HawkModel(cfg)
        opt = torch.optim.AdamW(model.parameters(), lr=1e-4)

        def step():
            with torch.autocast(device_type="cuda", dtype=torch.bfloat16):
                loss = model(ids, ids)
            loss.backward()
            opt.step()
            opt.zero_grad(set_to_none=True)
            return loss

        for _ in range(args.warmup):
            step()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            loss = step()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) * 1e3 / args.steps, float(loss.detach())

    def time_graph_steps():
        """The same step (forward, backward, AdamW) captured once in a HIP graph and replayed."""
        torch.manual_seed(args.seed)
        cfg = hk.HawkConfig(vocab_size=vocab, hidden_size=512, intermediate_size=1024, num_hidden_layers=8,
                            recurrent_size=512, num_blocks=16, conv_width=4)
        with torch.device(dev):
            model = hk.HawkModel(cfg)
        opt = torch.optim.AdamW(model.parameters(), lr=1e-4, capturable=True)

        def step():
            with torch.autocast(device_type="cuda", dtype=torch.bfloat16):
                loss = model(ids, ids)
            loss.backward()
            opt.step()
            return loss

        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(3):
                step()
                opt.zero_grad(set_to_none=True)
        torch.cuda.current_stream().wait_stream(side)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            static_loss = step()
        # the three eager steps above count as warm-up, so that every leg has taken the same
        # number of optimiser steps when its loss is read
        for _ in range(max(args.warmup - 3, 0)):
            graph.replay()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            graph.replay()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) * 1e3 / args.steps, float(static_loss.detach())

    fused_ms, fused_loss = time_steps()
    nodes_ms, nodes_loss = time_steps(fused_block_core=False)
    plain_ms, plain_loss = time_steps(fused_gates=False, fused_epilogue=False)
    graph_ms, graph_loss = time_graph_steps()
    return {
        "metric": "Hawk training step tokens/s (README model, batch 1 x 2048, bf16 autocast), 1 GPU",
        "value": B * T / (fused_ms * 1e-3), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": fused_ms, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16 autocast, f32 parameters and recurrence arithmetic",
        "data": f"synthetic, seed {args.seed}: random-init weights, token ids uniform in [1, {vocab})",
        "config": {"workload": "model: README Hawk (V=32000, H=R=512, I=1024, L=8, 16 blocks, conv 4), "
                               "forward + backward + AdamW, eager launches", "B": B, "T": T},
        "ms_per_step_with_conv_and_core_as_separate_nodes": nodes_ms,
        "ms_per_step_without_fused_gates_and_epilogue": plain_ms,
        "ms_per_step_as_hip_graph": graph_ms,
        "tokens_per_s_as_hip_graph": B * T / (graph_ms * 1e-3),
        "loss_after_last_step": {"fused": fused_loss, "separate_nodes": nodes_loss, "unfused": plain_loss,
                                 "hip_graph": graph_loss},
        "optimizer_steps_before_that_loss": {"fused": args.warmup + args.steps - 1,
                                             "separate_nodes": args.warmup + args.steps - 1,
                                             "unfused": args.warmup + args.steps - 1,
                                             "hip_graph": max(args.warmup, 3) + args.steps - 1},
        "roofline": None,
    }


def run_decode(args, lib, dev):
    """Decode at batch 256: tokens/s of whole model steps, and the hot path's share of a layer."""
    import hawk_pytorch_amd as hk
    from hawk_pytorch_amd import _lib

    B, prompt_len, vocab = 256, 1024, 32000
    cfg = hk.HawkConfig(vocab_size=vocab, hidden_size=2560, intermediate_size=7680, num_hidden_layers=26,
                        recurrent_size=2560, num_blocks=10, conv_width=4)
    torch.manual_seed(args.seed)
    with torch.device(dev):
        model = hk.HawkModel(cfg, use_cache=True)
    model.eval().bfloat16()
    for layer in model.layers:
        r = layer.recc
        # the recurrence's own parameters stay fp32 (the kernels read them as fp32)
        for p in (r.rg_lru_a_param, r.conv1d.w, r.conv1d.b, r.rg_lru_input_gate.b, r.rg_lru_a_gate.b):
            p.data = p.data.float()
        r.conv1d.out_dtype = torch.bfloat16
        torch.nn.init.normal_(r.resid_proj.weight, std=0.02)
        torch.nn.init.normal_(layer.mlp.resid_proj.weight, std=0.02)
    torch.nn.init.normal_(model.lm_head.weight, std=0.02)

    gen = torch.Generator(device=dev).manual_seed(args.seed)
    prompt = torch.randint(1, vocab, (B, prompt_len), device=dev, generator=gen)
    tok = torch.randint(1, vocab, (B, 1), device=dev, generator=gen)
    caches = model.new_cache(B)
    # weights are bf16 already, so autocast only rounds the few fp32 activations (the gate
    # logits pick up an fp32 bias) before the GEMMs; it casts no weight
    with torch.no_grad(), torch.autocast(device_type="cuda", dtype=torch.bfloat16):
        logits, caches = model(prompt, layer_past=caches)
        del logits
        for _ in range(args.warmup):
            model(tok, layer_past=caches)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            model(tok, layer_past=caches)
        torch.cuda.synchronize()
        eager_ms = (time.perf_counter() - t0) * 1e3 / args.steps

        graph = torch.cuda.CUDAGraph()
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            model(tok, layer_past=caches)
        torch.cuda.current_stream().wait_stream(side)
        with torch.cuda.graph(graph):
            static_logits, _ = model(tok, layer_past=caches)
        for _ in range(args.warmup):
            graph.replay()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            graph.replay()
        torch.cuda.synchronize()
        graph_ms = (time.perf_counter() - t0) * 1e3 / args.steps
        finite = bool(torch.isfinite(static_logits.float()).all())

    # The recurrent core of one layer and token through the C ABI, as `Hawk.forward` launches it:
    # hawk_decode_core_step_ws (window roll + conv, both gate projections, biases, recurrence,
    # output gate, both cache updates, one launch), every layer with its own weights and caches.
    D, W, nb, L = 2560, 4, 10, 26
    bw = D // nb
    bf, code = torch.bfloat16, _lib.HAWK_DTYPE_BF16
    xy = torch.randn(B, 2 * D, device=dev).to(bf)
    cw, cb = torch.randn(W, D, device=dev) * 0.5, torch.zeros(D, device=dev)
    bi, ba = torch.zeros(D, device=dev), torch.zeros(D, device=dev)
    lam = lambda_for_a8_range(torch.Generator().manual_seed(args.seed), D, 0.9, 0.999).to(dev)
    out = torch.empty(B, D, device=dev, dtype=bf)
    per_layer = [dict(conv_state=torch.randn(B, W - 1, D, device=dev).to(bf),
                      state=torch.zeros(B, D, device=dev).to(bf),
                      w_i=(torch.randn(nb, bw, bw, device=dev) * bw ** -0.5).to(bf),
                      w_a=(torch.randn(nb, bw, bw, device=dev) * bw ** -0.5).to(bf)) for _ in range(L)]
    core_ws = torch.zeros(max(lib.hawk_decode_core_workspace_bytes(B, D, nb), 4), dtype=torch.uint8, device=dev)

    def layer_core(p):
        stream = torch.cuda.current_stream(dev).cuda_stream
        _lib.check("decode_core_step_ws", lib.hawk_decode_core_step_ws(
            p["conv_state"].data_ptr(), xy.data_ptr(), 2 * D, cw.data_ptr(), cb.data_ptr(), p["w_i"].data_ptr(),
            bi.data_ptr(), p["w_a"].data_ptr(), ba.data_ptr(), lam.data_ptr(), xy.data_ptr() + 2 * D, 2 * D,
            p["state"].data_ptr(), out.data_ptr(), B, D, nb, W, code, code, code, core_ws.data_ptr(),
            core_ws.numel(), stream))

    # the two elementwise launches of the hot path alone (no projections), for comparison
    xn, y = xy[:, :D].contiguous(), xy[:, D:]
    u, xg, ag = (torch.randn(B, D, device=dev).to(bf) for _ in range(3))

    def layer_two_launches(p):
        stream = torch.cuda.current_stream(dev).cuda_stream
        _lib.check("conv1d_step", lib.hawk_conv1d_step(p["conv_state"].data_ptr(), xn.data_ptr(), cw.data_ptr(),
                                                       cb.data_ptr(), u.data_ptr(), B, D, W, code, code, stream))
        _lib.check("rglru_step_gated", lib.hawk_rglru_step_gated(
            u.data_ptr(), xg.data_ptr(), ag.data_ptr(), bi.data_ptr(), ba.data_ptr(), lam.data_ptr(), y.data_ptr(),
            2 * D, p["state"].data_ptr(), None, out.data_ptr(), B, D, code, code, stream))

    def graph_us_per_layer_step(fn):
        # 26 layers' launches as one HIP graph, so that the figure is the GPU's time and not the
        # host's launch rate
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            fn(per_layer[0])
        torch.cuda.current_stream().wait_stream(side)
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            for p in per_layer:
                fn(p)
        for _ in range(5):
            g.replay()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        n_rep = 40
        e0.record()
        for _ in range(n_rep):
            g.replay()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) * 1e3 / (n_rep * L)

    hot_us = graph_us_per_layer_step(layer_core)
    two_us = graph_us_per_layer_step(layer_two_launches)
    # core: conv window read and rewritten (3 + 3 rows), x_new, y, state read and written, out
    # (bf16), both gates' weights (bf16) and the fp32 vectors (conv taps and bias, gate biases, Lambda)
    hot_bytes = 11 * 2 * B * D + 2 * nb * bw * bw * 2 + (W + 4) * D * 4
    gbs = hot_bytes / (hot_us * 1e-6) / 1e9
    # two launches: conv step reads 3 state rows + new row, writes y and 3 rows; RG-LRU step reads
    # u, two logits, state, y, writes state and out  (bf16)
    two_bytes = (4 + 4 + 7) * 2 * B * D

    out_json = {
        "metric": "decode tokens/s, batch 256, 1 GPU (whole model step; hot path reported beside it)",
        "value": B / (graph_ms * 1e-3),
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": graph_ms,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16 weights and activations, f32 recurrence arithmetic",
        "data": f"synthetic, seed {args.seed}: random-init weights, random {prompt_len}-token prompt, vocabulary {vocab}",
        "config": {"workload": "decode: 26 layers, R=H=2560, I=7680, 10 gate blocks, B=256, one token per step",
                   "B": B, "layers": 26, "D": D, "vocab": vocab, "prompt": prompt_len},
        "eager_ms_per_step": eager_ms,
        "graph_ms_per_step": graph_ms,
        "logits_finite": finite,
        "hot_path_us_per_layer_step": hot_us,
        "roofline": {
            "bound": "hbm",
            "kernel": "decode_core_kernel via hawk_decode_core_step_ws (one launch per layer and token, the "
                      "path Hawk.forward takes; each of the 26 layers has its own weights; launch-bound)",
            "achieved": gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": gbs / HBM_PEAK_GBS, "traffic": None,
            "algorithmic_bytes_per_launch": hot_bytes, "launch_us": hot_us,
        },
        "two_elementwise_launches": {
            "kernel": "conv1d_step_kernel + rglru_step_kernel (no projections; two launches per layer and token)",
            "us_per_layer_step": two_us, "algorithmic_bytes": two_bytes,
            "GBs": two_bytes / (two_us * 1e-6) / 1e9,
        },
    }
    return out_json


def run_scan(args, lib, dev, name, steps, warmup, settle, calibration_copy=False):
    """Times `steps` forward + backward steps of scan workload `name`; returns the record."""
    from hawk_pytorch_amd import _lib

    B, T, D, (lo, hi), with_conv = WORKLOADS[name]
    N = B * T * D
    code = _lib.HAWK_DTYPE_BF16
    bf = torch.bfloat16

    mixed = name == "scan_mixed"
    in_dt = torch.float32 if mixed else bf
    in_code = _lib.HAWK_DTYPE_F32 if mixed else code
    gen = torch.Generator(device=dev).manual_seed(args.seed)
    x, xg, ag = (act_randn(args, (B, T, D), in_dt, dev, gen) for _ in range(3))
    gout = act_randn(args, (B, T, D), bf, dev, gen)
    lam = lambda_for_a8_range(torch.Generator().manual_seed(args.seed), D, lo, hi).to(dev)
    h = act_empty(args, (B, T, D), bf, dev)
    dx, dxg, dag = (act_empty(args, (B, T, D), in_dt, dev) for _ in range(3))
    dlam = torch.empty(D, dtype=torch.float32, device=dev)
    ws = torch.zeros(lib.hawk_scan_workspace_bytes(B, T, D, in_code), dtype=torch.uint8, device=dev)
    if with_conv:
        W = 4
        cw = (torch.randn(W, D, device=dev, generator=gen) * 0.5).float()
        cb = torch.zeros(D, device=dev)
        u = act_empty(args, (B, T, D), in_dt, dev)       # conv output, the scan's x
        du = act_empty(args, (B, T, D), in_dt, dev)      # conv input gradient
        dw = torch.empty(W, D, device=dev)
        db = torch.empty(D, device=dev)
        cws = torch.empty(lib.hawk_conv1d_bwd_workspace_bytes(B, T, D, W), dtype=torch.uint8, device=dev)
    gated = name == "scan_gated"
    if gated:
        xy = act_randn(args, (B, T, 2 * D), bf, dev, gen)
        y = xy[..., D:]               # the gate half of the block's input projection, in place
        gated_out = act_empty(args, (B, T, D), bf, dev)
        dy = act_empty(args, (B, T, D), bf, dev)
    stream = torch.cuda.current_stream(dev).cuda_stream

    def fwd():
        if gated:
            _lib.check("scan_gated_fwd", lib.hawk_rglru_scan_gated_fwd(
                x.data_ptr(), xg.data_ptr(), ag.data_ptr(), lam.data_ptr(), y.data_ptr(), 2 * D, h.data_ptr(),
                gated_out.data_ptr(), None, B, T, D, code, code, ws.data_ptr(), ws.numel(), stream))
            return
        if mixed:
            _lib.check("scan_fwd_mixed", lib.hawk_rglru_scan_fwd_mixed(
                x.data_ptr(), xg.data_ptr(), ag.data_ptr(), lam.data_ptr(), h.data_ptr(), B, T, D, in_code, code,
                ws.data_ptr(), ws.numel(), stream))
            return
        src = x
        if with_conv:
            _lib.check("conv_fwd", lib.hawk_conv1d_fwd(x.data_ptr(), cw.data_ptr(), cb.data_ptr(), None,
                                                       u.data_ptr(), B, T, D, W, code, code, stream))
            src = u
        _lib.check("scan_fwd", lib.hawk_rglru_scan_fwd(src.data_ptr(), xg.data_ptr(), ag.data_ptr(),
                                                       lam.data_ptr(), h.data_ptr(), B, T, D, code,
                                                       ws.data_ptr(), ws.numel(), stream))

    def bwd():
        if gated:
            _lib.check("scan_gated_bwd", lib.hawk_rglru_scan_gated_bwd(
                x.data_ptr(), xg.data_ptr(), ag.data_ptr(), lam.data_ptr(), y.data_ptr(), 2 * D, h.data_ptr(),
                gout.data_ptr(), dx.data_ptr(), dxg.data_ptr(), dag.data_ptr(), dy.data_ptr(), D, dlam.data_ptr(),
                B, T, D, code, code, ws.data_ptr(), ws.numel(), stream))
            return
        if mixed:
            _lib.check("scan_bwd_mixed", lib.hawk_rglru_scan_bwd_mixed(
                x.data_ptr(), xg.data_ptr(), ag.data_ptr(), lam.data_ptr(), h.data_ptr(), gout.data_ptr(),
                dx.data_ptr(), dxg.data_ptr(), dag.data_ptr(), dlam.data_ptr(), B, T, D, in_code, code,
                ws.data_ptr(), ws.numel(), stream))
            return
        src = u if with_conv else x
        _lib.check("scan_bwd", lib.hawk_rglru_scan_bwd(src.data_ptr(), xg.data_ptr(), ag.data_ptr(),
                                                       lam.data_ptr(), h.data_ptr(), gout.data_ptr(),
                                                       dx.data_ptr(), dxg.data_ptr(), dag.data_ptr(),
                                                       dlam.data_ptr(), B, T, D, code, ws.data_ptr(),
                                                       ws.numel(), stream))

    def conv_bwd():
        _lib.check("conv_bwd", lib.hawk_conv1d_bwd(dx.data_ptr(), x.data_ptr(), cw.data_ptr(), du.data_ptr(),
                                                   dw.data_ptr(), db.data_ptr(), B, T, D, W, code, code,
                                                   cws.data_ptr(), cws.numel(), stream))

    if calibration_copy:
        for _ in range(3):
            h.copy_(x)  # reads 2*N bytes, writes 2*N bytes
        torch.cuda.synchronize()

    for _ in range(settle + warmup):
        fwd()
        bwd()
        if with_conv:
            conv_bwd()
    torch.cuda.synchronize()

    # Timed region: `steps` steps, nothing but the launches between one event (and one host clock
    # reading) before and one after.  An event recorded between two launches costs the GPU 3-4 us
    # (a marker packet that the next dispatch waits behind), which a training loop does not pay.
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    start.record()
    for k in range(steps):
        fwd()
        bwd()
        if with_conv:
            conv_bwd()
    end.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    region_gpu_ms = start.elapsed_time(end)

    # Launch durations: the same `steps` steps again, right behind the timed region, now with an
    # event after every launch.  The forward launch of step k runs from the end of step k-1 (its
    # last event) to the first event of step k; two events bracket the backward launch.
    ev = [[torch.cuda.Event(enable_timing=True) for _ in range(3 if with_conv else 2)] for _ in range(steps)]
    start = torch.cuda.Event(enable_timing=True)
    start.record()
    for k in range(steps):
        fwd()
        ev[k][0].record()
        bwd()
        ev[k][1].record()
        if with_conv:
            conv_bwd()
            ev[k][2].record()
    torch.cuda.synchronize()

    flag = ctypes.c_int(0)
    _lib.check("status", lib.hawk_scan_workspace_status(ws.data_ptr(), stream, ctypes.byref(flag)))
    if flag.value != 0:
        print("bench.py: a scan tile gave up waiting for its carry; results are invalid", file=sys.stderr)
        sys.exit(1)

    step_end = [start] + [e[-1] for e in ev]
    fwd_ms = float(np.mean([step_end[k].elapsed_time(ev[k][0]) for k in range(steps)]))
    bwd_ms = float(np.mean([e[0].elapsed_time(e[1]) for e in ev]))
    ms_per_step = wall * 1e3 / steps
    ms_per_step_with_events = step_end[0].elapsed_time(step_end[-1]) / steps
    elem = 2  # bytes per bf16 activation element
    # gated: the forward also reads y and writes out; the backward also reads y and writes dy
    fwd_bytes = (6 if gated else 4) * elem * N + (2 * elem * N if with_conv else 0)
    bwd_bytes = (10 if gated else 8) * elem * N
    if mixed:  # three fp32 inputs + bf16 h; three fp32 inputs + bf16 h, grad_out, three fp32 gradients
        fwd_bytes, bwd_bytes = (3 * 4 + 2) * N, (3 * 4 + 2 + 2 + 3 * 4) * N
    step_bytes = fwd_bytes + bwd_bytes + (3 * elem * N if with_conv else 0)
    bwd_gbs = bwd_bytes / (bwd_ms * 1e-3) / 1e9

    traffic = measured_traffic(name)
    out = {
        "metric": "RG-LRU scan fwd+bwd tokens/s and achieved HBM GB/s (% of peak), 1 GPU",
        "value": B * T / (ms_per_step * 1e-3),
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": steps,
        "warmup": warmup,
        "settle_steps": settle,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": ("f32 inputs and gradients, bf16 h and grad_out, f32 state and accumulation" if mixed
                  else "bf16 in/out, f32 state and accumulation"),
        "data": f"synthetic, seed {args.seed}: x, gate logits, grad ~ N(0,1); a^8 ~ U({lo},{hi})",
        "config": {
            "workload": f"{name}: RG-LRU scan"
                        + (" + temporal conv1d (W=4)" if with_conv else "")
                        + (" fused with out = gelu(y) * h" if gated else "")
                        + f" fwd+bwd, B={B}, T={T}, D={D}, " + ("f32 in / bf16 state" if mixed else "bf16")
                        + f"; {settle} + {warmup} untimed steps before the {steps} timed ones",
            "B": B, "T": T, "D": D,
            "allocation": ALLOCATION[bool(args.plain_alloc)],
        },
        "timed_region": {"steps": steps, "host_ms": wall * 1e3, "gpu_ms_between_events": region_gpu_ms,
                         "events_inside": 0},
        "launch_timing_region": {"steps": steps, "events_per_step": 3 if with_conv else 2,
                                 "ms_per_step": ms_per_step_with_events,
                                 "note": "the same steps run again right behind the timed region with an event "
                                         "after every launch; roofline and fwd come from here"},
        "roofline": {
            "bound": "hbm",
            "kernel": "rglru_scan_bwd_kernel" + (" (gated)" if gated else "")
                      + " (+ dlam_reduce_kernel, same launch call)",
            "achieved": bwd_gbs,
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": bwd_gbs / HBM_PEAK_GBS,
            "traffic": traffic,
            # the same launch time against the HBM bytes rocprofv3 counted for this launch (the
            # algorithmic bytes plus the carry words): what "achieved HBM bandwidth in rocprof" reads
            "traffic_frac": None if traffic is None else traffic / (bwd_ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
            "algorithmic_bytes_per_launch": bwd_bytes,
            "launch_ms": bwd_ms,
        },
        "fwd": {"ms": fwd_ms, "GBs": fwd_bytes / (fwd_ms * 1e-3) / 1e9,
                "frac": fwd_bytes / (fwd_ms * 1e-3) / 1e9 / HBM_PEAK_GBS},
        "step_hbm": {"GBs": step_bytes / (ms_per_step * 1e-3) / 1e9,
                     "frac": step_bytes / (ms_per_step * 1e-3) / 1e9 / HBM_PEAK_GBS},
    }
    out["_cpu_args"] = (B, D, lo, hi)
    out["_buffers"] = {"x": x, "xg": xg, "ag": ag, "h": h, "gout": gout, "dx": dx, "dxg": dxg, "dag": dag}
    return out


def run_stream_ceiling(buf, steps, settle):
    """Stock PyTorch streaming kernels on the scan's own operands, timed like the scan's launches.

    What a plain elementwise kernel with the forward's and the backward's read/write mix reaches on
    this box in this process: the scale against which the scan's GB/s can be read."""
    x, xg, ag, h, gout, dx, dxg, dag = (buf[k] for k in ("x", "xg", "ag", "h", "gout", "dx", "dxg", "dag"))
    nbytes = x.numel() * x.element_size()

    def copy_1r1w():
        h.copy_(x)

    def addcmul_3r1w():
        torch.addcmul(x, xg, ag, out=h)

    def composition_5r3w():
        torch.addcmul(x, xg, ag, out=dx)   # 3 reads, 1 write
        torch.mul(h, gout, out=dxg)        # 2 reads, 1 write
        dag.fill_(0.5)                     # 1 write

    # The library's own streaming probes: copies with the scan kernels' memory instructions, flat
    # (16 KiB of every tensor per workgroup) and in the scan's workgroup shape (eight waves stacked
    # in time on 16 rows x 256 bytes each), for the forward's and the backward's mix.
    from hawk_pytorch_amd import _lib

    lib = _lib.load()
    stream = torch.cuda.current_stream(x.device).cuda_stream
    row_pitch = x.shape[-1] * x.element_size()
    seq_groups = x.shape[1] // 128   # 128-row tiles per sequence: the probe then walks tiles in the scan's launch order

    def probe(reads, writes, shape):
        r = (ctypes.c_void_p * len(reads))(*[t.data_ptr() for t in reads])
        w = (ctypes.c_void_p * len(writes))(*[t.data_ptr() for t in writes])

        def call():
            _lib.check("stream_probe", lib.hawk_stream_probe(r, len(reads), w, len(writes), nbytes, row_pitch, shape,
                                                             stream))
        return call

    fwd_mix, bwd_mix = ((x, xg, ag), (h,)), ((x, xg, ag, h, gout), (dx, dxg, dag))
    rec = {}
    for name, fn, tensors, kernels in (("copy_1r1w", copy_1r1w, 2, 1), ("addcmul_3r1w", addcmul_3r1w, 4, 1),
                                       ("composition_5r3w", composition_5r3w, 8, 3),
                                       ("probe_flat_3r1w", probe(*fwd_mix, 0), 4, 1),
                                       ("probe_flat_5r3w", probe(*bwd_mix, 0), 8, 1),
                                       ("probe_scan_shape_3r1w", probe(*fwd_mix, 1), 4, 1),
                                       ("probe_scan_shape_5r3w", probe(*bwd_mix, 1), 8, 1),
                                       ("probe_scan_order_3r1w", probe(*fwd_mix, seq_groups), 4, 1),
                                       ("probe_scan_order_5r3w", probe(*bwd_mix, seq_groups), 8, 1)):
        for _ in range(settle):
            fn()
        torch.cuda.synchronize()
        # per call, as the scan's launches are timed: an event after every call
        ev = [torch.cuda.Event(enable_timing=True) for _ in range(steps + 1)]
        ev[0].record()
        for k in range(steps):
            fn()
            ev[k + 1].record()
        torch.cuda.synchronize()
        with_events_ms = ev[0].elapsed_time(ev[-1]) / steps
        # and back to back, as the timed region runs
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for k in range(steps):
            fn()
        b.record()
        torch.cuda.synchronize()
        ms = a.elapsed_time(b) / steps
        moved = tensors * nbytes
        rec[name] = {"kernels": kernels, "bytes": moved, "us": ms * 1e3, "GBs": moved / (ms * 1e-3) / 1e9,
                     "frac": moved / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
                     "us_with_an_event_per_call": with_events_ms * 1e3,
                     "frac_with_an_event_per_call": moved / (with_events_ms * 1e-3) / 1e9 / HBM_PEAK_GBS}
    rec["note"] = ("torch.Tensor.copy_, torch.addcmul(out=) and addcmul + mul + fill_ on the headline's x, x_rg_lru, "
                   "a_rg_lru, h, grad_out and gradient tensors (bf16, %d MB each), and the library's copy kernels "
                   "(hawk_stream_probe: non-temporal buffer loads and stores; flat = 16 KiB of every tensor per "
                   "workgroup, scan_shape = eight waves stacked in time on 16 rows x 256 bytes each, as a scan "
                   "workgroup reads its tile, tiles in memory order; scan_order = the same tiles in the order the "
                   "scan's launch takes them: position along the sequence slowest, then batch row, then channel "
                   "tile) on the same tensors; %d settling calls, then %d timed calls; frac is "
                   "of the 8 TB/s peak" % (nbytes // 1000000, settle, steps))
    return rec


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=10, help="untimed steps before the timed ones")
    ap.add_argument("--settle-steps", type=int, default=100,
                    help="further untimed steps run before the warm-up in the kernel workloads (scan*, long, gates, "
                         "block): kernel durations settle about 50 steps (20 ms) after the GPU leaves idle")
    ap.add_argument("--fp32-gate-weights", action="store_true",
                    help="workload gates: hand the projection kernels the fp32 weights instead of rounding them "
                         "to bf16 once per step")
    ap.add_argument("--unfused-conv", action="store_true",
                    help="workload block: the single entry points (two weight casts, conv and gate projections as "
                         "two launches on a copy of the x half of the input projection, gradients into separate "
                         "tensors, a closing reduction per backward call) instead of one host call per direction "
                         "on the projection's output in place")
    ap.add_argument("--plain-alloc", action="store_true",
                    help="kernel workloads: allocate every tensor with a plain torch.empty (large blocks then start "
                         "on 2 MiB boundaries) instead of the library's placement of activation tensors, bases "
                         "256 bytes apart modulo 1 KiB")
    ap.add_argument("--workload", choices=sorted(WORKLOADS) + ["block", "decode", "gates", "model"], default="scan")
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-also", action="store_true",
                    help="default workload only: skip the sub-records for the long and scan_conv configurations")
    ap.add_argument("--record-traffic", nargs=3, metavar=("FETCH_BYTES", "WRITE_BYTES", "NOTE"),
                    help="no GPU run: store a measured HBM traffic figure for --workload in "
                         "profiles/hbm_traffic.json, stamped with the digest of the present kernel sources")
    ap.add_argument("--calibration-copy", action="store_true",
                    help="also run three plain device-to-device copies of one activation tensor (outside the "
                         "timed region) so that a rocprofv3 --pmc run has a kernel of known traffic to scale "
                         "FETCH_SIZE / WRITE_SIZE by")
    args = ap.parse_args()

    if args.record_traffic:
        record_traffic(args.workload, float(args.record_traffic[0]), float(args.record_traffic[1]),
                       args.record_traffic[2])
        return
    if args.gpus != 1:
        print("bench.py: this build runs on exactly one GPU (the path needs no collective); "
              "--gpus must be 1", file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; the HIP kernels have no CPU fallback", file=sys.stderr)
        sys.exit(1)

    from hawk_pytorch_amd import _lib

    lib = _lib.load()
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    others = {"decode": run_decode, "gates": run_gates, "model": run_model, "block": run_block}
    if args.workload in others:
        print(json.dumps(others[args.workload](args, lib, dev)))
        return
    out = run_scan(args, lib, dev, args.workload, args.steps, args.warmup, args.settle_steps, args.calibration_copy)
    cpu_args = out.pop("_cpu_args")
    buffers = out.pop("_buffers")
    if args.workload == "scan":
        # the streaming ceiling of this box, in this process, on the same tensors
        ceiling = run_stream_ceiling(buffers, max(20, args.steps // 4), max(10, args.settle_steps // 4))
        ceiling["scan_fwd_over_addcmul_3r1w"] = (out["fwd"]["GBs"]
                                                 / (ceiling["addcmul_3r1w"]["bytes"]
                                                    / (ceiling["addcmul_3r1w"]["us_with_an_event_per_call"] * 1e-6) / 1e9))
        ceiling["scan_bwd_over_composition_5r3w"] = (out["roofline"]["achieved"]
                                                     / (ceiling["composition_5r3w"]["bytes"]
                                                        / (ceiling["composition_5r3w"]["us_with_an_event_per_call"] * 1e-6) / 1e9))
        ceiling["scan_step_over_both"] = ((ceiling["addcmul_3r1w"]["us"] + ceiling["composition_5r3w"]["us"]) * 1e-3
                                          / out["ms_per_step"])
        # the same three ratios against the library's copy kernels in the scan's own workgroup shape
        ceiling["scan_fwd_over_probe_scan_shape_3r1w"] = (
            ceiling["probe_scan_shape_3r1w"]["us_with_an_event_per_call"] * 1e-3 / out["fwd"]["ms"])
        ceiling["scan_bwd_over_probe_scan_shape_5r3w"] = (
            ceiling["probe_scan_shape_5r3w"]["us_with_an_event_per_call"] * 1e-3 / out["roofline"]["launch_ms"])
        ceiling["scan_step_over_probe_scan_shape"] = (
            (ceiling["probe_scan_shape_3r1w"]["us"] + ceiling["probe_scan_shape_5r3w"]["us"]) * 1e-3
            / out["ms_per_step"])
        # ... and against the same copies with the tiles taken in the scan's launch order
        ceiling["scan_fwd_over_probe_scan_order_3r1w"] = (
            ceiling["probe_scan_order_3r1w"]["us_with_an_event_per_call"] * 1e-3 / out["fwd"]["ms"])
        ceiling["scan_bwd_over_probe_scan_order_5r3w"] = (
            ceiling["probe_scan_order_5r3w"]["us_with_an_event_per_call"] * 1e-3 / out["roofline"]["launch_ms"])
        ceiling["scan_step_over_probe_scan_order"] = (
            (ceiling["probe_scan_order_3r1w"]["us"] + ceiling["probe_scan_order_5r3w"]["us"]) * 1e-3
            / out["ms_per_step"])
        ceiling["scan_step_over_probe_flat"] = (
            (ceiling["probe_flat_3r1w"]["us"] + ceiling["probe_flat_5r3w"]["us"]) * 1e-3 / out["ms_per_step"])
        out["stream_ceiling"] = ceiling
    del buffers
    if args.workload == "scan" and not args.no_also:
        # the other scan configurations of the benchmark definition, timed after the headline
        # region in the same process (fewer steps; the GPU is already at its steady clocks)
        also = {}
        few = argparse.Namespace(**vars(args))
        few.steps, few.settle_steps, few.calibration_copy = max(20, args.steps // 4), max(10, args.settle_steps // 4), False
        plain = argparse.Namespace(**vars(args))
        plain.plain_alloc = not args.plain_alloc
        for other in ("scan", "long", "scan_conv", "scan_gated"):
            torch.cuda.empty_cache()
            # the headline's shape once more with the other placement of its tensors
            rec = run_scan(plain if other == "scan" else args, lib, dev, other, few.steps, args.warmup,
                           few.settle_steps)
            rec.pop("_cpu_args")
            rec.pop("_buffers")
            key = ("scan_plain_alloc" if plain.plain_alloc else "scan_library_alloc") if other == "scan" else other
            also[key] = {k: rec[k] for k in ("config", "value", "unit", "ms_per_step", "steps", "warmup",
                                             "settle_steps", "roofline", "fwd", "step_hbm")}
        # the matrix-core gate projections and the recurrent core of one layer at the same shape, and
        # one-token decode steps of the 26-layer model at batch 256, and training steps of the README model
        for other, fn in (("gates", run_gates), ("block", run_block), ("decode", run_decode), ("model", run_model)):
            torch.cuda.empty_cache()
            rec = fn(few, lib, dev)
            also[other] = {k: rec[k] for k in rec if k not in ("metric", "n_gpus", "higher_is_better", "scaling",
                                                              "vs_baseline", "dtype", "data") and rec[k] is not None}
        out["also"] = also
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(*cpu_args, args.seed)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
