"""Direct ctypes calls into libhawk_hip.so for the GPU tests: raw device pointers, sizes
and a stream, exactly what a non-Python host would pass.  No torch op wrappers involved."""

import ctypes

import numpy as np
import torch

from hawk_pytorch_amd import _lib

TORCH_DTYPE = {"f32": torch.float32, "bf16": torch.bfloat16}


def to_dev(a, dtype):
    return torch.from_numpy(np.ascontiguousarray(a)).to(device="cuda", dtype=TORCH_DTYPE[dtype]).contiguous()


def to_np(t):
    return t.detach().float().cpu().numpy().astype(np.float64)


def _stream():
    return torch.cuda.current_stream().cuda_stream


def new_workspace(B, T, D, dtype, through_init=True):
    lib = _lib.load()
    n = lib.hawk_scan_workspace_bytes(B, T, D, _lib.dtype_code(TORCH_DTYPE[dtype]))
    assert n > 0
    if through_init:
        ws = torch.empty(n, dtype=torch.uint8, device="cuda")
        ws.fill_(0xAB)  # garbage, so that the init call is what zeroes it
        _lib.check("hawk_scan_workspace_init", lib.hawk_scan_workspace_init(ws.data_ptr(), n, _stream()))
    else:
        ws = torch.zeros(n, dtype=torch.uint8, device="cuda")
    return ws


def workspace_flag(ws):
    flag = ctypes.c_int(-1)
    _lib.check("hawk_scan_workspace_status",
               _lib.load().hawk_scan_workspace_status(ws.data_ptr(), _stream(), ctypes.byref(flag)))
    return flag.value


def scan_fwd(x, xg, ag, lam, ws=None):
    """x, xg, ag: device tensors [B,T,D] (bf16 or fp32); lam: device fp32 [D]."""
    B, T, D = x.shape
    h = torch.empty_like(x)
    if ws is None:
        ws = new_workspace(B, T, D, "bf16" if x.dtype == torch.bfloat16 else "f32")
    rc = _lib.load().hawk_rglru_scan_fwd(
        x.data_ptr(), xg.data_ptr(), ag.data_ptr(), lam.data_ptr(), h.data_ptr(), B, T, D,
        _lib.dtype_code(x.dtype), ws.data_ptr(), ws.numel(), _stream())
    _lib.check("hawk_rglru_scan_fwd", rc)
    return h


def scan_fwd_mixed(x, xg, ag, lam, out_dtype, ws=None):
    """Inputs in x.dtype, h in out_dtype (the (f32, bf16) pair is the interesting one)."""
    B, T, D = x.shape
    h = torch.empty((B, T, D), dtype=out_dtype, device="cuda")
    if ws is None:
        ws = new_workspace(B, T, D, "bf16" if x.dtype == torch.bfloat16 else "f32")
    rc = _lib.load().hawk_rglru_scan_fwd_mixed(
        x.data_ptr(), xg.data_ptr(), ag.data_ptr(), lam.data_ptr(), h.data_ptr(), B, T, D,
        _lib.dtype_code(x.dtype), _lib.dtype_code(out_dtype), ws.data_ptr(), ws.numel(), _stream())
    _lib.check("hawk_rglru_scan_fwd_mixed", rc)
    return h


def scan_bwd_mixed(x, xg, ag, lam, h, gout, ws=None):
    """x, xg, ag and the returned gradients in x.dtype; h and gout in h.dtype."""
    B, T, D = x.shape
    dx, dxg, dag = torch.empty_like(x), torch.empty_like(x), torch.empty_like(x)
    dlam = torch.empty(D, dtype=torch.float32, device="cuda")
    if ws is None:
        ws = new_workspace(B, T, D, "bf16" if x.dtype == torch.bfloat16 else "f32")
    rc = _lib.load().hawk_rglru_scan_bwd_mixed(
        x.data_ptr(), xg.data_ptr(), ag.data_ptr(), lam.data_ptr(), h.data_ptr(), gout.data_ptr(),
        dx.data_ptr(), dxg.data_ptr(), dag.data_ptr(), dlam.data_ptr(), B, T, D,
        _lib.dtype_code(x.dtype), _lib.dtype_code(h.dtype), ws.data_ptr(), ws.numel(), _stream())
    _lib.check("hawk_rglru_scan_bwd_mixed", rc)
    return dx, dxg, dag, dlam


def scan_bwd(x, xg, ag, lam, h, gout, ws=None):
    B, T, D = x.shape
    dx, dxg, dag = torch.empty_like(x), torch.empty_like(x), torch.empty_like(x)
    dlam = torch.empty(D, dtype=torch.float32, device="cuda")
    if ws is None:
        ws = new_workspace(B, T, D, "bf16" if x.dtype == torch.bfloat16 else "f32")
    rc = _lib.load().hawk_rglru_scan_bwd(
        x.data_ptr(), xg.data_ptr(), ag.data_ptr(), lam.data_ptr(), h.data_ptr(), gout.data_ptr(),
        dx.data_ptr(), dxg.data_ptr(), dag.data_ptr(), dlam.data_ptr(), B, T, D,
        _lib.dtype_code(x.dtype), ws.data_ptr(), ws.numel(), _stream())
    _lib.check("hawk_rglru_scan_bwd", rc)
    return dx, dxg, dag, dlam


def conv_fwd(x, w, b, state=None, y_dtype=None):
    B, T, D = x.shape
    W = w.shape[0]
    y_dtype = y_dtype or x.dtype
    y = torch.empty((B, T, D), dtype=y_dtype, device="cuda")
    rc = _lib.load().hawk_conv1d_fwd(
        x.data_ptr(), w.data_ptr(), b.data_ptr(), None if state is None else state.data_ptr(), y.data_ptr(),
        B, T, D, W, _lib.dtype_code(x.dtype), _lib.dtype_code(y_dtype), _stream())
    _lib.check("hawk_conv1d_fwd", rc)
    return y


def conv_bwd(gy, x, w):
    B, T, D = x.shape
    W = w.shape[0]
    lib = _lib.load()
    dx = torch.empty_like(x)
    dw = torch.empty((W, D), dtype=torch.float32, device="cuda")
    db = torch.empty((D,), dtype=torch.float32, device="cuda")
    n = lib.hawk_conv1d_bwd_workspace_bytes(B, T, D, W)
    ws = torch.empty(n, dtype=torch.uint8, device="cuda")
    rc = lib.hawk_conv1d_bwd(
        gy.data_ptr(), x.data_ptr(), w.data_ptr(), dx.data_ptr(), dw.data_ptr(), db.data_ptr(), B, T, D, W,
        _lib.dtype_code(x.dtype), _lib.dtype_code(gy.dtype), ws.data_ptr(), n, _stream())
    _lib.check("hawk_conv1d_bwd", rc)
    return dx, dw, db


def conv_fwd_strided(x, w, b, y, state=None):
    """x, y: [B,T,D] views with unit channel stride and evenly spaced rows; y is written in place."""
    B, T, D = x.shape
    assert x.stride(2) == 1 and y.stride(2) == 1 and x.stride(0) == T * x.stride(1) and y.stride(0) == T * y.stride(1)
    rc = _lib.load().hawk_conv1d_fwd_strided(
        x.data_ptr(), x.stride(1), w.data_ptr(), b.data_ptr(), None if state is None else state.data_ptr(),
        y.data_ptr(), y.stride(1), B, T, D, w.shape[0], _lib.dtype_code(x.dtype), _lib.dtype_code(y.dtype), _stream())
    _lib.check("hawk_conv1d_fwd_strided", rc)
    return y


def conv_bwd_strided(gy, x, w, dx):
    """x, dx: [B,T,D] views with evenly spaced rows (dx is written in place); gy dense."""
    B, T, D = x.shape
    W = w.shape[0]
    lib = _lib.load()
    assert x.stride(2) == 1 and dx.stride(2) == 1 and x.stride(0) == T * x.stride(1) and dx.stride(0) == T * dx.stride(1)
    dw = torch.empty((W, D), dtype=torch.float32, device="cuda")
    db = torch.empty((D,), dtype=torch.float32, device="cuda")
    n = lib.hawk_conv1d_bwd_workspace_bytes(B, T, D, W)
    ws = torch.empty(n, dtype=torch.uint8, device="cuda")
    rc = lib.hawk_conv1d_bwd_strided(
        gy.data_ptr(), x.data_ptr(), x.stride(1), w.data_ptr(), dx.data_ptr(), dx.stride(1), dw.data_ptr(),
        db.data_ptr(), B, T, D, W, _lib.dtype_code(x.dtype), _lib.dtype_code(gy.dtype), ws.data_ptr(), n, _stream())
    _lib.check("hawk_conv1d_bwd_strided", rc)
    return dw, db


def conv_step(state, x_new, w, b, y_dtype=None):
    B, D = x_new.shape
    W = w.shape[0]
    y_dtype = y_dtype or x_new.dtype
    y = torch.empty((B, D), dtype=y_dtype, device="cuda")
    rc = _lib.load().hawk_conv1d_step(
        state.data_ptr(), x_new.data_ptr(), w.data_ptr(), b.data_ptr(), y.data_ptr(), B, D, W,
        _lib.dtype_code(x_new.dtype), _lib.dtype_code(y_dtype), _stream())
    _lib.check("hawk_conv1d_step", rc)
    return y


def rglru_step(x, xg, ag, lam, state):
    B, D = x.shape
    h = torch.empty_like(x)
    rc = _lib.load().hawk_rglru_step(
        x.data_ptr(), xg.data_ptr(), ag.data_ptr(), lam.data_ptr(), state.data_ptr(), h.data_ptr(), B, D,
        _lib.dtype_code(x.dtype), _lib.dtype_code(state.dtype), _stream())
    _lib.check("hawk_rglru_step", rc)
    return h


def scan_gated_fwd(x, xg, ag, lam, y, out_dtype=None, want_h=True, want_last=True, ws=None):
    """y: [B,T,D] view with unit channel stride and evenly spaced rows (may be a slice of a
    wider tensor).  Returns (out, h or None, h_last or None)."""
    B, T, D = x.shape
    out_dtype = out_dtype or x.dtype
    assert y.dtype == out_dtype and y.stride(2) == 1
    ldy = y.stride(1) if T > 1 else (y.stride(0) if B > 1 else D)
    assert B == 1 or y.stride(0) == T * ldy
    out = torch.empty((B, T, D), dtype=out_dtype, device="cuda")
    h = torch.empty((B, T, D), dtype=out_dtype, device="cuda") if want_h else None
    h_last = torch.full((B, D), float("nan"), dtype=out_dtype, device="cuda") if want_last else None
    if ws is None:
        ws = new_workspace(B, T, D, "bf16" if x.dtype == torch.bfloat16 else "f32")
    rc = _lib.load().hawk_rglru_scan_gated_fwd(
        x.data_ptr(), xg.data_ptr(), ag.data_ptr(), lam.data_ptr(), y.data_ptr(), ldy,
        _lib.ptr(h), out.data_ptr(), _lib.ptr(h_last), B, T, D, _lib.dtype_code(x.dtype),
        _lib.dtype_code(out_dtype), ws.data_ptr(), ws.numel(), _stream())
    _lib.check("hawk_rglru_scan_gated_fwd", rc)
    return out, h, h_last


def scan_gated_bwd(x, xg, ag, lam, y, h, gout, dy=None, ws=None):
    """dy: optional preallocated [B,T,D] view with evenly spaced rows to receive the gate's gradient."""
    B, T, D = x.shape
    assert y.dtype == h.dtype and gout.dtype == h.dtype
    ldy = y.stride(1) if T > 1 else (y.stride(0) if B > 1 else D)
    dx, dxg, dag = torch.empty_like(x), torch.empty_like(x), torch.empty_like(x)
    if dy is None:
        dy = torch.empty((B, T, D), dtype=h.dtype, device="cuda")
    lddy = dy.stride(1) if T > 1 else (dy.stride(0) if B > 1 else D)
    dlam = torch.empty(D, dtype=torch.float32, device="cuda")
    if ws is None:
        ws = new_workspace(B, T, D, "bf16" if x.dtype == torch.bfloat16 else "f32")
    rc = _lib.load().hawk_rglru_scan_gated_bwd(
        x.data_ptr(), xg.data_ptr(), ag.data_ptr(), lam.data_ptr(), y.data_ptr(), ldy, h.data_ptr(),
        gout.data_ptr(), dx.data_ptr(), dxg.data_ptr(), dag.data_ptr(), dy.data_ptr(), lddy, dlam.data_ptr(),
        B, T, D, _lib.dtype_code(x.dtype), _lib.dtype_code(h.dtype), ws.data_ptr(), ws.numel(), _stream())
    _lib.check("hawk_rglru_scan_gated_bwd", rc)
    return dx, dxg, dag, dlam, dy


def rglru_step_gated(x, xg, ag, bias_i, bias_a, lam, y, state, want_h=True):
    """y: [B,D] view with unit channel stride (rows may be further apart than D)."""
    B, D = x.shape
    h = torch.empty_like(x) if want_h else None
    out = torch.empty_like(x)
    rc = _lib.load().hawk_rglru_step_gated(
        x.data_ptr(), xg.data_ptr(), ag.data_ptr(), _lib.ptr(bias_i), _lib.ptr(bias_a), lam.data_ptr(),
        y.data_ptr(), y.stride(0) if B > 1 else D, state.data_ptr(), _lib.ptr(h), out.data_ptr(), B, D,
        _lib.dtype_code(x.dtype), _lib.dtype_code(state.dtype), _stream())
    _lib.check("hawk_rglru_step_gated", rc)
    return out, h


def gate_proj_fwd(x, w_i, b_i, w_a, b_a, out_dtype=None):
    """x [M,D] (bf16/fp32), w_* [nb,bw,bw] (bf16/fp32), b_* [D] fp32 or None."""
    M, D = x.shape
    nb = w_i.shape[0]
    out_dtype = out_dtype or x.dtype
    oi = torch.empty((M, D), dtype=out_dtype, device="cuda")
    oa = torch.empty((M, D), dtype=out_dtype, device="cuda")
    rc = _lib.load().hawk_gate_proj_fwd(
        x.data_ptr(), w_i.data_ptr(), _lib.ptr(b_i), w_a.data_ptr(), _lib.ptr(b_a), oi.data_ptr(), oa.data_ptr(),
        M, D, nb, _lib.dtype_code(x.dtype), _lib.dtype_code(w_i.dtype), _lib.dtype_code(out_dtype), _stream())
    _lib.check("hawk_gate_proj_fwd", rc)
    return oi, oa


def conv_gate_proj_fwd(x, conv_w, conv_b, w_i, b_i, w_a, b_a):
    """x [B,T,D] bf16 with unit channel stride and dense batch/time (rows may be further apart
    than D); returns the conv output and both logits, dense [B,T,D] bf16."""
    B, T, D = x.shape
    assert x.stride(2) == 1 and x.stride(0) == T * x.stride(1)
    nb = w_i.shape[0]
    u, oi, oa = (torch.empty((B, T, D), dtype=torch.bfloat16, device="cuda") for _ in range(3))
    rc = _lib.load().hawk_conv_gate_proj_fwd(
        x.data_ptr(), x.stride(1), conv_w.data_ptr(), conv_b.data_ptr(), w_i.data_ptr(), _lib.ptr(b_i),
        w_a.data_ptr(), _lib.ptr(b_a), u.data_ptr(), oi.data_ptr(), oa.data_ptr(), B, T, D, nb, conv_w.shape[0],
        _lib.dtype_code(w_i.dtype), _stream())
    _lib.check("hawk_conv_gate_proj_fwd", rc)
    return u, oi, oa


def decode_core_step(conv_state, x_new, conv_w, conv_b, w_i, b_i, w_a, b_a, lam, y, state, ws=None):
    """x_new, y: [B,D] bf16 views with unit channel stride (rows may be further apart than D);
    conv_state [B,W-1,D] bf16 and state [B,D] are updated in place.  Returns out [B,D] bf16.
    ws: zeroed counters (uint8 tensor) for the entry point that cuts a block over workgroups."""
    B, D = x_new.shape
    W = conv_w.shape[0]
    out = torch.empty((B, D), dtype=torch.bfloat16, device="cuda")
    args = [
        _lib.ptr(conv_state), x_new.data_ptr(), x_new.stride(0) if B > 1 else D, conv_w.data_ptr(), conv_b.data_ptr(),
        w_i.data_ptr(), _lib.ptr(b_i), w_a.data_ptr(), _lib.ptr(b_a), lam.data_ptr(), y.data_ptr(),
        y.stride(0) if B > 1 else D, state.data_ptr(), out.data_ptr(), B, D, w_i.shape[0], W,
        _lib.dtype_code(x_new.dtype), _lib.dtype_code(w_i.dtype), _lib.dtype_code(state.dtype)]
    if ws is None:
        rc = _lib.load().hawk_decode_core_step(*args, _stream())
        _lib.check("hawk_decode_core_step", rc)
    else:
        rc = _lib.load().hawk_decode_core_step_ws(*args, ws.data_ptr(), ws.numel(), _stream())
        _lib.check("hawk_decode_core_step_ws", rc)
    return out


def decode_core_workspace(B, D, nb):
    n = _lib.load().hawk_decode_core_workspace_bytes(B, D, nb)
    assert n > 0
    return torch.zeros(n, dtype=torch.uint8, device="cuda")


def gate_proj_bwd_input(dxg, dag, w_i, w_a, dx_dtype=None, addend=None, in_place=False):
    """addend: optional [M,D] tensor of dx's dtype added to the result; in_place writes over it."""
    M, D = dxg.shape
    nb = w_i.shape[0]
    dx_dtype = dx_dtype or dxg.dtype
    dx = addend if in_place else torch.empty((M, D), dtype=dx_dtype, device="cuda")
    rc = _lib.load().hawk_gate_proj_bwd_input(
        dxg.data_ptr(), dag.data_ptr(), w_i.data_ptr(), w_a.data_ptr(), _lib.ptr(addend), dx.data_ptr(), M, D, nb,
        _lib.dtype_code(dxg.dtype), _lib.dtype_code(w_i.dtype), _lib.dtype_code(dx_dtype), _stream())
    _lib.check("hawk_gate_proj_bwd_input", rc)
    return dx


def gate_proj_bwd_weights(x, dxg, dag, nb, with_bias=True):
    M, D = x.shape
    bw = D // nb
    lib = _lib.load()
    n = lib.hawk_gate_proj_bwd_weights_workspace_bytes(M, D, nb)
    assert n > 0
    ws = torch.full((n,), 0xAB, dtype=torch.uint8, device="cuda")  # garbage: the kernels must not rely on zeros
    dwi = torch.empty((nb, bw, bw), dtype=torch.float32, device="cuda")
    dwa = torch.empty_like(dwi)
    dbi = torch.empty(D, dtype=torch.float32, device="cuda") if with_bias else None
    dba = torch.empty(D, dtype=torch.float32, device="cuda") if with_bias else None
    rc = lib.hawk_gate_proj_bwd_weights(
        x.data_ptr(), dxg.data_ptr(), dag.data_ptr(), dwi.data_ptr(), _lib.ptr(dbi), dwa.data_ptr(), _lib.ptr(dba),
        M, D, nb, _lib.dtype_code(x.dtype), _lib.dtype_code(dxg.dtype), ws.data_ptr(), n, _stream())
    _lib.check("hawk_gate_proj_bwd_weights", rc)
    return dwi, dbi, dwa, dba


def gate_weights_to_bf16(w_i, w_a):
    nb, bw, _ = w_i.shape
    oi, oa = (torch.empty((nb, bw, bw), dtype=torch.bfloat16, device="cuda") for _ in range(2))
    rc = _lib.load().hawk_gate_weights_to_bf16(w_i.data_ptr(), w_a.data_ptr(), oi.data_ptr(), oa.data_ptr(), nb, bw,
                                               _stream())
    _lib.check("hawk_gate_weights_to_bf16", rc)
    return oi, oa


def block_core_fwd(xy, conv_w, conv_b, w_i, b_i, w_a, b_a, lam, round_weights=True, want_h=True, want_last=True,
                   ws=None):
    """xy [B,T,2D] bf16 with unit channel stride and dense batch/time.  Returns
    (out, u, xg, ag, h or None, h_last or None, w16 or None)."""
    B, T, D2 = xy.shape
    D = D2 // 2
    assert xy.stride(2) == 1 and xy.stride(0) == T * xy.stride(1)
    nb, bw, _ = w_i.shape
    e = lambda: torch.empty((B, T, D), dtype=torch.bfloat16, device="cuda")  # noqa: E731
    u, xg, ag, out = e(), e(), e(), e()
    h = e() if want_h else None
    h_last = torch.full((B, D), float("nan"), dtype=torch.bfloat16, device="cuda") if want_last else None
    w16 = None
    if round_weights and w_i.dtype == torch.float32:
        w16 = torch.full((2, nb, bw, bw), float("nan"), dtype=torch.bfloat16, device="cuda")
    if ws is None:
        ws = new_workspace(B, T, D, "bf16")
    rc = _lib.load().hawk_block_core_fwd(
        xy.data_ptr(), xy.stride(1), conv_w.data_ptr(), conv_b.data_ptr(), w_i.data_ptr(), _lib.ptr(b_i),
        w_a.data_ptr(), _lib.ptr(b_a), _lib.dtype_code(w_i.dtype), _lib.ptr(w16), lam.data_ptr(), u.data_ptr(),
        xg.data_ptr(), ag.data_ptr(), _lib.ptr(h), out.data_ptr(), _lib.ptr(h_last), B, T, D, nb, conv_w.shape[0],
        ws.data_ptr(), ws.numel(), _stream())
    _lib.check("hawk_block_core_fwd", rc)
    return out, u, xg, ag, h, h_last, w16


def block_core_bwd(xy, u, xg, ag, h, conv_w, w_i, w_a, lam, gout, with_bias=True, ws=None):
    """Returns (d_xy, d_conv_w, d_conv_b, dw_i, db_i, dw_a, db_a, dlam, du)."""
    B, T, D2 = xy.shape
    D = D2 // 2
    nb, bw, _ = w_i.shape
    W = conv_w.shape[0]
    lib = _lib.load()
    d_xy = torch.full((B, T, D2), float("nan"), dtype=torch.bfloat16, device="cuda")
    du, dxg, dag = (torch.empty((B, T, D), dtype=torch.bfloat16, device="cuda") for _ in range(3))
    f = lambda *s: torch.full(s, float("nan"), dtype=torch.float32, device="cuda")  # noqa: E731
    dcw, dcb, dwi, dwa, dlam = f(W, D), f(D), f(nb, bw, bw), f(nb, bw, bw), f(D)
    dbi, dba = (f(D), f(D)) if with_bias else (None, None)
    if ws is None:
        ws = new_workspace(B, T, D, "bf16")
    garbage = lambda n: torch.full((max(n, 16),), 0xAB, dtype=torch.uint8, device="cuda")  # noqa: E731
    gws = garbage(lib.hawk_gate_proj_bwd_weights_workspace_bytes(B * T, D, nb))
    cws = garbage(lib.hawk_conv1d_bwd_workspace_bytes(B, T, D, W))
    rc = lib.hawk_block_core_bwd(
        xy.data_ptr(), xy.stride(1), u.data_ptr(), xg.data_ptr(), ag.data_ptr(), h.data_ptr(), conv_w.data_ptr(),
        w_i.data_ptr(), w_a.data_ptr(), _lib.dtype_code(w_i.dtype), lam.data_ptr(), gout.data_ptr(), d_xy.data_ptr(),
        D2, du.data_ptr(), dxg.data_ptr(), dag.data_ptr(), dcw.data_ptr(), dcb.data_ptr(), dwi.data_ptr(),
        _lib.ptr(dbi), dwa.data_ptr(), _lib.ptr(dba), dlam.data_ptr(), B, T, D, nb, W, ws.data_ptr(), ws.numel(),
        gws.data_ptr(), gws.numel(), cws.data_ptr(), cws.numel(), _stream())
    _lib.check("hawk_block_core_bwd", rc)
    return d_xy, dcw, dcb, dwi, dbi, dwa, dba, dlam, du
