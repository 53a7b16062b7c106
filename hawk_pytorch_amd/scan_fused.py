"""RG-LRU linear scan operator backed by the gfx950 HIP kernels.

Public surface mirrors the upstream operator boundary (hawk/scan_fused.py:319-445):

    sequential_scan_forward(x, x_rg_lru, a_rg_lru, a_param) -> h
    sequential_scan_backward(x, x_rg_lru, a_rg_lru, a_param, h_saved, grad_out)
        -> (dx, dx_rg_lru, da_rg_lru, da_param)
    DiagonalRecurrence            torch.autograd.Function
    fused_linear_scan             = DiagonalRecurrence.apply

and, beyond upstream, the scan fused with the block's gate (hawk/hawk.py:134-135, :186):

    fused_linear_scan_gated(x, x_rg_lru, a_rg_lru, a_param, y) -> gelu(y) * h

Differences from upstream, all deliberate:

* Under autocast, fp32 activations are NOT first cast to bf16 by three extra kernels
  (upstream: ``custom_fwd(cast_inputs=bfloat16)``, scan_fused.py:428): mixed-precision
  kernels read fp32, keep fp32 state, write bf16 ``h``, and return fp32 gradients.
* Lambda (``a_param``) and its gradient stay fp32 even under autocast (upstream's
  ``custom_fwd(cast_inputs=bfloat16)`` rounds Lambda to bf16 too, scan_fused.py:428).
* fp32 activations are stored as fp32 (upstream rounds every store through bf16,
  scan_fused.py:81, :109, :194-196).
* T == 1 works (upstream's backward needs T >= 2, scan_fused.py:133).

The kernels are reached through ``torch.library`` custom ops so that ``torch.compile``
traces through the call without a graph break.
"""

from __future__ import annotations

import warnings
from typing import Tuple

import torch
from torch.autograd import Function

from . import _lib

BLOCKSIZE = 64  # upstream's channel-block contract: D must be a multiple of this


def _prepare(*tensors: torch.Tensor):
    return tuple(t if t.is_contiguous() else t.contiguous() for t in tensors)


def _launch_scan_fwd(x, x_rg_lru, a_rg_lru, a_param, h_bf16: bool) -> torch.Tensor:
    dev = _lib.require_cuda(x, x_rg_lru, a_rg_lru, a_param)
    x, x_rg_lru, a_rg_lru, a_param = (_lib.dense16(t) for t in (x, x_rg_lru, a_rg_lru, a_param))
    b, sq, d = x.shape
    in_code = _lib.dtype_code(x.dtype)
    out_dtype = torch.bfloat16 if h_bf16 else x.dtype
    lib = _lib.load()
    h = _lib.activation_empty((b, sq, d), out_dtype, dev)
    nbytes = lib.hawk_scan_workspace_bytes(b, sq, d, in_code)
    ws = _lib.scan_workspace(dev, nbytes)
    with torch.cuda.device(dev):
        status = lib.hawk_rglru_scan_fwd_mixed(
            x.data_ptr(), x_rg_lru.data_ptr(), a_rg_lru.data_ptr(), a_param.data_ptr(), h.data_ptr(),
            b, sq, d, in_code, _lib.dtype_code(out_dtype), ws.data_ptr(), ws.numel(), _lib.stream_ptr(dev),
        )
    _lib.check("hawk_rglru_scan_fwd_mixed", status)
    return h


def _launch_scan_bwd(x, x_rg_lru, a_rg_lru, a_param, h_saved, grad_out):
    dev = _lib.require_cuda(x, x_rg_lru, a_rg_lru, a_param, h_saved, grad_out)
    x, x_rg_lru, a_rg_lru, a_param, h_saved, grad_out = (
        _lib.dense16(t) for t in (x, x_rg_lru, a_rg_lru, a_param, h_saved, grad_out)
    )
    b, sq, d = x.shape
    in_code = _lib.dtype_code(x.dtype)
    lib = _lib.load()
    dx, dxg, dag = (_lib.activation_empty(x.shape, x.dtype, dev) for _ in range(3))
    dlam = torch.empty(d, dtype=torch.float32, device=dev)
    nbytes = lib.hawk_scan_workspace_bytes(b, sq, d, in_code)
    ws = _lib.scan_workspace(dev, nbytes)
    with torch.cuda.device(dev):
        status = lib.hawk_rglru_scan_bwd_mixed(
            x.data_ptr(), x_rg_lru.data_ptr(), a_rg_lru.data_ptr(), a_param.data_ptr(),
            h_saved.data_ptr(), grad_out.data_ptr(), dx.data_ptr(), dxg.data_ptr(), dag.data_ptr(),
            dlam.data_ptr(), b, sq, d, in_code, _lib.dtype_code(h_saved.dtype),
            ws.data_ptr(), ws.numel(), _lib.stream_ptr(dev),
        )
    _lib.check("hawk_rglru_scan_bwd_mixed", status)
    return dx, dxg, dag, dlam


# ---------------------------------------------------------------------------------------
# torch.library registration (opaque to Dynamo, with shape/dtype propagation rules).
# x, x_rg_lru, a_rg_lru share a dtype (bf16 or fp32); h is bf16 when h_bf16 is set, else
# that same dtype; in the backward h_saved and grad_out share h's dtype and the three
# activation gradients come back in the inputs' dtype.
# ---------------------------------------------------------------------------------------
@torch.library.custom_op("hawk_amd::rglru_scan_fwd", mutates_args=(), device_types="cuda")
def _rglru_scan_fwd_op(
    x: torch.Tensor, x_rg_lru: torch.Tensor, a_rg_lru: torch.Tensor, a_param: torch.Tensor, h_bf16: bool
) -> torch.Tensor:
    return _launch_scan_fwd(x, x_rg_lru, a_rg_lru, a_param, h_bf16)


@_rglru_scan_fwd_op.register_fake
def _(x, x_rg_lru, a_rg_lru, a_param, h_bf16):
    return torch.empty(x.shape, dtype=torch.bfloat16 if h_bf16 else x.dtype, device=x.device)


@torch.library.custom_op("hawk_amd::rglru_scan_bwd", mutates_args=(), device_types="cuda")
def _rglru_scan_bwd_op(
    x: torch.Tensor,
    x_rg_lru: torch.Tensor,
    a_rg_lru: torch.Tensor,
    a_param: torch.Tensor,
    h_saved: torch.Tensor,
    grad_out: torch.Tensor,
) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    return _launch_scan_bwd(x, x_rg_lru, a_rg_lru, a_param, h_saved, grad_out)


@_rglru_scan_bwd_op.register_fake
def _(x, x_rg_lru, a_rg_lru, a_param, h_saved, grad_out):
    e = lambda: torch.empty_like(x, memory_format=torch.contiguous_format)  # noqa: E731
    return e(), e(), e(), torch.empty(x.shape[-1], dtype=torch.float32, device=x.device)


# ---------------------------------------------------------------------------------------
# Upstream-shaped host wrappers
# ---------------------------------------------------------------------------------------
def _check_shapes(x, x_rg_lru, a_rg_lru, a_param):
    assert x.dim() == 3, f"Error: expected x of shape [b, sq, d], got {tuple(x.shape)}"
    assert x_rg_lru.shape == x.shape and a_rg_lru.shape == x.shape, (
        "Error: x, x_rg_lru and a_rg_lru must have the same shape, got "
        f"{tuple(x.shape)}, {tuple(x_rg_lru.shape)}, {tuple(a_rg_lru.shape)}"
    )
    d = x.shape[-1]
    assert d % BLOCKSIZE == 0, f"Error: expected model dimension to be a multiple of {BLOCKSIZE}"
    assert a_param.shape == (d,), f"Error: expected a_param of shape [{d}], got {tuple(a_param.shape)}"
    assert x_rg_lru.dtype == x.dtype and a_rg_lru.dtype == x.dtype, (
        f"Error: x, x_rg_lru and a_rg_lru must share a dtype, got {x.dtype}, {x_rg_lru.dtype}, {a_rg_lru.dtype}"
    )


def sequential_scan_forward(
    x: torch.Tensor,
    x_rg_lru: torch.Tensor,
    a_rg_lru: torch.Tensor,  # [b,sq,d]
    a_param: torch.Tensor,  # [d]
    out_dtype: torch.dtype | None = None,
) -> torch.Tensor:
    """Forward pass of the RG-LRU scan (drop-in for hawk/scan_fused.py:319-360).

    Non-contiguous inputs are silently copied, as upstream does; D must be a multiple of
    64, as upstream asserts.  ``a_param`` is used in fp32 whatever dtype it arrives in.
    ``out_dtype=torch.bfloat16`` with fp32 inputs selects the mixed-precision kernel
    (fp32 read, bf16 h) that replaces upstream's cast-then-scan sequence.
    """
    _check_shapes(x, x_rg_lru, a_rg_lru, a_param)
    x, x_rg_lru, a_rg_lru = _prepare(x, x_rg_lru, a_rg_lru)
    a_param = a_param.float().contiguous()
    h_bf16 = out_dtype == torch.bfloat16 or (out_dtype is None and x.dtype == torch.bfloat16)
    assert out_dtype in (None, x.dtype, torch.bfloat16), f"unsupported h dtype {out_dtype} for {x.dtype} inputs"
    return _rglru_scan_fwd_op(x, x_rg_lru, a_rg_lru, a_param, h_bf16)


def sequential_scan_backward(
    x_saved: torch.Tensor,
    x_rg_lru_saved: torch.Tensor,
    a_rg_lru_saved: torch.Tensor,
    a_param_saved: torch.Tensor,
    h_saved: torch.Tensor,
    grad_out: torch.Tensor,
) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    """Backward pass of the RG-LRU scan (drop-in for hawk/scan_fused.py:363-424).

    Returns (dx, dx_rg_lru, da_rg_lru, da_param[D]); the three activation gradients have
    the dtype of the saved inputs, da_param is fp32 and already summed over the batch.
    ``h_saved`` may be bf16 while the inputs are fp32 (mixed-precision forward).  A
    non-contiguous ``grad_out`` is copied with a warning, as upstream.
    """
    _check_shapes(x_saved, x_rg_lru_saved, a_rg_lru_saved, a_param_saved)
    assert h_saved.shape == x_saved.shape and grad_out.shape == x_saved.shape
    if not grad_out.is_contiguous():
        grad_out = grad_out.contiguous()
        warnings.warn(
            "`grad_out` tensor is not contiguous. Setting to contiguous and attempting to continue. "
            "This may impact runtime."
        )
    if h_saved.dtype not in (x_saved.dtype, torch.bfloat16):
        h_saved = h_saved.to(x_saved.dtype)
    if grad_out.dtype != h_saved.dtype:
        grad_out = grad_out.to(h_saved.dtype)
    x_saved, x_rg_lru_saved, a_rg_lru_saved, h_saved, grad_out = _prepare(
        x_saved, x_rg_lru_saved, a_rg_lru_saved, h_saved, grad_out
    )
    a_param_saved = a_param_saved.float().contiguous()
    return _rglru_scan_bwd_op(x_saved, x_rg_lru_saved, a_rg_lru_saved, a_param_saved, h_saved, grad_out)


def _common_input_dtype(*tensors: torch.Tensor) -> torch.dtype:
    """bf16 only if every activation already is bf16; fp32 otherwise (fp16/fp64 compute in fp32)."""
    if all(t.dtype == torch.bfloat16 for t in tensors):
        return torch.bfloat16
    return torch.float32


class DiagonalRecurrence(Function):
    """h = scan(x, x_rg_lru, a_rg_lru, a_param) with the hand-written reverse-time backward.

    Same four positional tensor arguments and four gradients as upstream
    (hawk/scan_fused.py:426-442).  Under CUDA autocast h is bf16, as with upstream's
    ``custom_fwd(cast_inputs=torch.bfloat16)``, but fp32 activations are not cast first:
    the mixed-precision kernels read them as fp32 and round in registers, and the backward
    writes their gradients directly in fp32.  Lambda is always used in fp32.
    """

    @staticmethod
    def forward(ctx, x, x_rg_lru, a_rg_lru, a_param) -> torch.Tensor:
        in_dtype = _common_input_dtype(x, x_rg_lru, a_rg_lru)
        xc, xgc, agc = (t if t.dtype == in_dtype else t.to(in_dtype) for t in (x, x_rg_lru, a_rg_lru))
        autocast = torch.is_autocast_enabled("cuda")
        h = sequential_scan_forward(xc, xgc, agc, a_param, torch.bfloat16 if autocast else None)
        ctx.save_for_backward(xc, xgc, agc, a_param, h)
        if not autocast and x.dtype not in (torch.bfloat16, torch.float32):
            return h.to(x.dtype)
        return h

    @staticmethod
    def backward(ctx, grad_output):  # type: ignore[override]
        (x, x_rg_lru, a_rg_lru, a_param, h_saved) = ctx.saved_tensors
        x_grad, x_rg_lru_grad, a_rg_lru_grad, a_param_grad = sequential_scan_backward(
            x, x_rg_lru, a_rg_lru, a_param, h_saved, grad_output
        )
        return x_grad, x_rg_lru_grad, a_rg_lru_grad, a_param_grad.to(a_param.dtype)


fused_linear_scan = DiagonalRecurrence.apply


# ---------------------------------------------------------------------------------------
# Scan fused with the block's gate: out = gelu(y) * h  (hawk/hawk.py:134-135 applied to the
# scan's result, :186).  y is usually one half of a wider projection, so it is taken in
# place when its rows are evenly spaced.
# ---------------------------------------------------------------------------------------
def _row_stride(t: torch.Tensor):
    """Elements between consecutive rows of a [B, T, D] tensor whose row r = b*T + t starts at
    r * stride, or None when t is not laid out that way."""
    b, sq, d = t.shape
    if t.stride(2) != 1 and d > 1:
        return None
    if sq > 1:
        ld = t.stride(1)
    elif b > 1:
        ld = t.stride(0)
    else:
        ld = d
    if ld < d or (b > 1 and t.stride(0) != sq * ld):
        return None
    return ld


def _launch_scan_gated_fwd(x, x_rg_lru, a_rg_lru, a_param, y, h_bf16: bool, want_h: bool, want_last: bool):
    dev = _lib.require_cuda(x, x_rg_lru, a_rg_lru, a_param, y)
    x, x_rg_lru, a_rg_lru, a_param = (_lib.dense16(t) for t in (x, x_rg_lru, a_rg_lru, a_param))
    b, sq, d = x.shape
    in_code = _lib.dtype_code(x.dtype)
    out_dtype = torch.bfloat16 if h_bf16 else x.dtype
    if y.dtype != out_dtype:
        y = y.to(out_dtype)
    ldy = _row_stride(y)
    if ldy is None:
        y = _lib.dense16(y)
        ldy = d
    lib = _lib.load()
    out = _lib.activation_empty((b, sq, d), out_dtype, dev)
    h = _lib.activation_empty((b, sq, d) if want_h else (0,), out_dtype, dev)
    h_last = torch.empty((b, 1, d) if want_last else (0,), dtype=out_dtype, device=dev)
    nbytes = lib.hawk_scan_workspace_bytes(b, sq, d, in_code)
    ws = _lib.scan_workspace(dev, nbytes)
    with torch.cuda.device(dev):
        status = lib.hawk_rglru_scan_gated_fwd(
            x.data_ptr(), x_rg_lru.data_ptr(), a_rg_lru.data_ptr(), a_param.data_ptr(), y.data_ptr(), ldy,
            h.data_ptr() if want_h else None, out.data_ptr(), h_last.data_ptr() if want_last else None,
            b, sq, d, in_code, _lib.dtype_code(out_dtype), ws.data_ptr(), ws.numel(), _lib.stream_ptr(dev),
        )
    _lib.check("hawk_rglru_scan_gated_fwd", status)
    return out, h, h_last


def _launch_scan_gated_bwd(x, x_rg_lru, a_rg_lru, a_param, y, h_saved, grad_out):
    dev = _lib.require_cuda(x, x_rg_lru, a_rg_lru, a_param, y, h_saved, grad_out)
    x, x_rg_lru, a_rg_lru, a_param, h_saved, grad_out = (
        _lib.dense16(t) for t in (x, x_rg_lru, a_rg_lru, a_param, h_saved, grad_out)
    )
    b, sq, d = x.shape
    in_code = _lib.dtype_code(x.dtype)
    if y.dtype != h_saved.dtype:
        y = y.to(h_saved.dtype)
    ldy = _row_stride(y)
    if ldy is None:
        y = _lib.dense16(y)
        ldy = d
    lib = _lib.load()
    dx, dxg, dag = (_lib.activation_empty(x.shape, x.dtype, dev) for _ in range(3))
    dy = _lib.activation_empty((b, sq, d), h_saved.dtype, dev)
    dlam = torch.empty(d, dtype=torch.float32, device=dev)
    nbytes = lib.hawk_scan_workspace_bytes(b, sq, d, in_code)
    ws = _lib.scan_workspace(dev, nbytes)
    with torch.cuda.device(dev):
        status = lib.hawk_rglru_scan_gated_bwd(
            x.data_ptr(), x_rg_lru.data_ptr(), a_rg_lru.data_ptr(), a_param.data_ptr(), y.data_ptr(), ldy,
            h_saved.data_ptr(), grad_out.data_ptr(), dx.data_ptr(), dxg.data_ptr(), dag.data_ptr(),
            dy.data_ptr(), d, dlam.data_ptr(), b, sq, d, in_code, _lib.dtype_code(h_saved.dtype),
            ws.data_ptr(), ws.numel(), _lib.stream_ptr(dev),
        )
    _lib.check("hawk_rglru_scan_gated_bwd", status)
    return dx, dxg, dag, dlam, dy


@torch.library.custom_op("hawk_amd::rglru_scan_gated_fwd", mutates_args=(), device_types="cuda")
def _rglru_scan_gated_fwd_op(
    x: torch.Tensor,
    x_rg_lru: torch.Tensor,
    a_rg_lru: torch.Tensor,
    a_param: torch.Tensor,
    y: torch.Tensor,
    h_bf16: bool,
    want_h: bool,
    want_last: bool,
) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    return _launch_scan_gated_fwd(x, x_rg_lru, a_rg_lru, a_param, y, h_bf16, want_h, want_last)


@_rglru_scan_gated_fwd_op.register_fake
def _(x, x_rg_lru, a_rg_lru, a_param, y, h_bf16, want_h, want_last):
    dt = torch.bfloat16 if h_bf16 else x.dtype
    b, sq, d = x.shape
    return (
        torch.empty((b, sq, d), dtype=dt, device=x.device),
        torch.empty((b, sq, d) if want_h else (0,), dtype=dt, device=x.device),
        torch.empty((b, 1, d) if want_last else (0,), dtype=dt, device=x.device),
    )


@torch.library.custom_op("hawk_amd::rglru_scan_gated_bwd", mutates_args=(), device_types="cuda")
def _rglru_scan_gated_bwd_op(
    x: torch.Tensor,
    x_rg_lru: torch.Tensor,
    a_rg_lru: torch.Tensor,
    a_param: torch.Tensor,
    y: torch.Tensor,
    h_saved: torch.Tensor,
    grad_out: torch.Tensor,
) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    return _launch_scan_gated_bwd(x, x_rg_lru, a_rg_lru, a_param, y, h_saved, grad_out)


@_rglru_scan_gated_bwd_op.register_fake
def _(x, x_rg_lru, a_rg_lru, a_param, y, h_saved, grad_out):
    e = lambda: torch.empty_like(x, memory_format=torch.contiguous_format)  # noqa: E731
    return (
        e(), e(), e(),
        torch.empty(x.shape[-1], dtype=torch.float32, device=x.device),
        torch.empty(x.shape, dtype=h_saved.dtype, device=x.device),
    )


class GatedDiagonalRecurrence(Function):
    """(out, h_last) = (gelu(y) * h, h[:, -1:]) with h = scan(x, x_rg_lru, a_rg_lru, a_param).

    One kernel per direction instead of the scan, a GELU and a product (and their three
    autograd mirrors).  Dtype rules are DiagonalRecurrence's; y and out have h's dtype.
    The state sequence h is written only when a gradient will be asked for; h_last (what
    the decode cache keeps, hawk/hawk.py:190) is not differentiable.
    """

    @staticmethod
    def forward(ctx, x, x_rg_lru, a_rg_lru, a_param, y, want_last):
        in_dtype = _common_input_dtype(x, x_rg_lru, a_rg_lru)
        xc, xgc, agc = (t if t.dtype == in_dtype else t.to(in_dtype) for t in (x, x_rg_lru, a_rg_lru))
        autocast = torch.is_autocast_enabled("cuda")
        _check_shapes(xc, xgc, agc, a_param)
        assert y.shape == x.shape, f"Error: expected y of shape {tuple(x.shape)}, got {tuple(y.shape)}"
        xc, xgc, agc = _prepare(xc, xgc, agc)
        lam = a_param.float().contiguous()
        h_bf16 = autocast or in_dtype == torch.bfloat16
        want_h = any(ctx.needs_input_grad[:5])
        out, h, h_last = _rglru_scan_gated_fwd_op(xc, xgc, agc, lam, y, h_bf16, want_h, bool(want_last))
        if want_h:
            ctx.save_for_backward(xc, xgc, agc, a_param, y, h)
        ctx.y_dtype = y.dtype
        ctx.mark_non_differentiable(h_last)
        if not autocast and x.dtype not in (torch.bfloat16, torch.float32):
            out, h_last = out.to(x.dtype), h_last.to(x.dtype)
        return out, h_last

    @staticmethod
    def backward(ctx, grad_out, _grad_last):  # type: ignore[override]
        (x, x_rg_lru, a_rg_lru, a_param, y, h_saved) = ctx.saved_tensors
        if not grad_out.is_contiguous():
            grad_out = grad_out.contiguous()
        if grad_out.dtype != h_saved.dtype:
            grad_out = grad_out.to(h_saved.dtype)
        dx, dxg, dag, dlam, dy = _rglru_scan_gated_bwd_op(
            x, x_rg_lru, a_rg_lru, a_param.float().contiguous(), y, h_saved, grad_out
        )
        if dy.dtype != ctx.y_dtype:
            dy = dy.to(ctx.y_dtype)
        return dx, dxg, dag, dlam.to(a_param.dtype), dy, None


def fused_linear_scan_gated(x, x_rg_lru, a_rg_lru, a_param, y, return_last_state: bool = False):
    """gelu(y) * fused_linear_scan(x, x_rg_lru, a_rg_lru, a_param) in one kernel per direction.

    With ``return_last_state`` also returns h[:, -1:, :] (shape [B, 1, D]), the recurrent
    state a decode cache keeps after prefill.
    """
    out, h_last = GatedDiagonalRecurrence.apply(x, x_rg_lru, a_rg_lru, a_param, y, return_last_state)
    return (out, h_last) if return_last_state else out


# ---------------------------------------------------------------------------------------
# The recurrent core of a Hawk block as one autograd node: both gate projections, the scan
# and the output gate (hawk/hawk.py:181-186 and :134-135).  Besides saving launches, one
# node lets the backward hand the scan's gradient of u to the projection kernel, which adds
# it to its own on the way out; as separate nodes autograd would sum the two in an extra
# pass over the tensor.
# ---------------------------------------------------------------------------------------
class RecurrentCore(Function):
    @staticmethod
    def forward(ctx, u, w_i, b_i, w_a, b_a, a_param, y, want_last):
        from .external import _gate_proj_fwd_op, kernel_weights  # deferred: external imports nothing from here

        assert u.dtype == torch.bfloat16, "the fused core runs on bf16 activations"
        uc = u if u.is_contiguous() else u.contiguous()
        lam = a_param.float().contiguous()
        ctx.dtypes = (w_i.dtype, b_i.dtype, w_a.dtype, b_a.dtype, a_param.dtype, y.dtype)
        w_i, w_a = kernel_weights(w_i, w_a, uc.numel() // uc.shape[-1])
        xg, ag = _gate_proj_fwd_op(uc, w_i, b_i.float().reshape(-1), w_a, b_a.float().reshape(-1), True)
        _check_shapes(uc, xg, ag, a_param)
        want_h = any(ctx.needs_input_grad[:7])
        out, h, h_last = _rglru_scan_gated_fwd_op(uc, xg, ag, lam, y, True, want_h, bool(want_last))
        if want_h:
            ctx.save_for_backward(uc, xg, ag, h, y, w_i, w_a, a_param)
        ctx.mark_non_differentiable(h_last)
        return out, h_last

    @staticmethod
    def backward(ctx, grad_out, _grad_last):  # type: ignore[override]
        from .external import _gate_proj_bwd_op

        u, xg, ag, h, y, w_i, w_a, a_param = ctx.saved_tensors
        go = grad_out if grad_out.dtype == h.dtype else grad_out.to(h.dtype)
        go = go if go.is_contiguous() else go.contiguous()
        du_scan, d_xg, d_ag, dlam, dy = _rglru_scan_gated_bwd_op(u, xg, ag, a_param.float().contiguous(), y, h, go)
        du, dw_i, db_i, dw_a, db_a = _gate_proj_bwd_op(u, d_xg, d_ag, w_i, w_a, du_scan)
        nb, bw, _ = w_i.shape
        t = ctx.dtypes
        return (du, dw_i.to(t[0]), db_i.reshape(nb, bw).to(t[1]), dw_a.to(t[2]), db_a.reshape(nb, bw).to(t[3]),
                dlam.to(t[4]), dy.to(t[5]), None)


def recurrent_core(u, input_gate, a_gate, a_param, y, return_last_state: bool = False):
    """``gelu(y) * scan(u, input_gate(u), a_gate(u), a_param)`` for bf16 ``u`` and gate modules
    the fused projection kernels serve (see ``external.gate_projections_supported``)."""
    out, h_last = RecurrentCore.apply(u, input_gate.w, input_gate.b, a_gate.w, a_gate.b, a_param, y,
                                      return_last_state)
    return (out, h_last) if return_last_state else out


# ---------------------------------------------------------------------------------------
# The same node with the temporal conv in front, fed by the block's input projection itself
# (hawk/hawk.py:163-186: chunk, Conv1D, both gates, scan, output gate).  xy is the [B,T,2D]
# output of that projection: the conv reads its first half and the output gate its second half
# in place (upstream's chunk gives views, but its Conv1D and scan copy them), the conv and both
# gate projections are one kernel, and the backward writes the two halves of the gradient of
# xy side by side into one tensor, where autograd would concatenate two.  One custom op per
# direction, so the host issues two calls per layer.
# ---------------------------------------------------------------------------------------
_FUSED_CONV_MIN_T = 32   # hawk_conv_gate_proj_fwd needs T >= 32 and a temporal width of 4


def block_core_layout_ok(xy: torch.Tensor) -> bool:
    """xy [B,T,2D] bf16 on the GPU with unit channel stride and evenly spaced rows a multiple of
    8 elements apart: what the kernels read in place.  (Plain Python on shapes and strides, so a
    tracing compiler sees through it.)"""
    if xy.dim() != 3 or xy.dtype != torch.bfloat16 or xy.device.type != "cuda" or xy.shape[-1] % 16 != 0:
        return False
    ld = _row_stride(xy)
    return ld is not None and ld % 8 == 0


def _launch_block_core_fwd(xy, conv_w, conv_b, w_i, b_i, w_a, b_a, lam, want_h: bool, want_last: bool):
    dev = _lib.require_cuda(xy, conv_w, conv_b, w_i, b_i, w_a, b_a, lam)
    if xy.data_ptr() % 16 != 0:
        xy = xy.clone(memory_format=torch.contiguous_format)
    B, T, D2 = xy.shape
    D = D2 // 2
    ld = _row_stride(xy)
    W = conv_w.shape[0]
    nb = w_i.shape[0]
    conv_w, conv_b, w_i, w_a, b_i, b_a, lam = (_lib.dense16(t) for t in (conv_w, conv_b, w_i, w_a, b_i, b_a, lam))
    bf, code = torch.bfloat16, _lib.HAWK_DTYPE_BF16
    u, xg, ag, out = (_lib.activation_empty((B, T, D), bf, dev) for _ in range(4))
    h = _lib.activation_empty((B, T, D) if want_h else (0,), bf, dev)
    h_last = torch.empty((B, 1, D) if want_last else (0,), dtype=bf, device=dev)
    lib = _lib.load()
    ws = _lib.scan_workspace(dev, lib.hawk_scan_workspace_bytes(B, T, D, code))
    y_ptr = xy.data_ptr() + D * xy.element_size()
    with torch.cuda.device(dev):
        st = _lib.stream_ptr(dev)
        if W == 4 and T >= _FUSED_CONV_MIN_T:
            # conv + both projections, then the gated scan: one host call
            _lib.check("hawk_block_core_fwd", lib.hawk_block_core_fwd(
                xy.data_ptr(), ld, conv_w.data_ptr(), conv_b.data_ptr(), w_i.data_ptr(), b_i.data_ptr(),
                w_a.data_ptr(), b_a.data_ptr(), _lib.dtype_code(w_i.dtype), None, lam.data_ptr(), u.data_ptr(),
                xg.data_ptr(), ag.data_ptr(), h.data_ptr() if want_h else None, out.data_ptr(),
                h_last.data_ptr() if want_last else None, B, T, D, nb, W, ws.data_ptr(), ws.numel(), st))
        else:
            _lib.check("hawk_conv1d_fwd_strided", lib.hawk_conv1d_fwd_strided(
                xy.data_ptr(), ld, conv_w.data_ptr(), conv_b.data_ptr(), None, u.data_ptr(), D, B, T, D, W, code,
                code, st))
            _lib.check("hawk_gate_proj_fwd", lib.hawk_gate_proj_fwd(
                u.data_ptr(), w_i.data_ptr(), b_i.data_ptr(), w_a.data_ptr(), b_a.data_ptr(), xg.data_ptr(),
                ag.data_ptr(), B * T, D, nb, code, _lib.dtype_code(w_i.dtype), code, st))
            _lib.check("hawk_rglru_scan_gated_fwd", lib.hawk_rglru_scan_gated_fwd(
                u.data_ptr(), xg.data_ptr(), ag.data_ptr(), lam.data_ptr(), y_ptr, ld,
                h.data_ptr() if want_h else None, out.data_ptr(), h_last.data_ptr() if want_last else None,
                B, T, D, code, code, ws.data_ptr(), ws.numel(), st))
    return out, u, xg, ag, h, h_last


def _launch_block_core_bwd(xy, u, xg, ag, h, conv_w, w_i, w_a, lam, grad_out):
    from .external import _gate_workspace  # deferred: external imports nothing from here

    dev = _lib.require_cuda(xy, u, xg, ag, h, conv_w, w_i, w_a, lam, grad_out)
    if xy.data_ptr() % 16 != 0:
        xy = xy.clone(memory_format=torch.contiguous_format)
    B, T, D2 = xy.shape
    D = D2 // 2
    ld = _row_stride(xy)
    W = conv_w.shape[0]
    nb, bw, _ = w_i.shape
    M = B * T
    conv_w, w_i, w_a, lam, grad_out = (_lib.dense16(t) for t in (conv_w, w_i, w_a, lam, grad_out))
    bf, code, f32 = torch.bfloat16, _lib.HAWK_DTYPE_BF16, torch.float32
    lib = _lib.load()
    d_xy = _lib.activation_empty((B, T, D2), bf, dev)
    du, dxg, dag = (_lib.activation_empty((B, T, D), bf, dev) for _ in range(3))
    dlam = torch.empty(D, dtype=f32, device=dev)
    dw_i, dw_a = (torch.empty((nb, bw, bw), dtype=f32, device=dev) for _ in range(2))
    db_i, db_a, dcb = (torch.empty(D, dtype=f32, device=dev) for _ in range(3))
    dcw = torch.empty((W, D), dtype=f32, device=dev)
    ws = _lib.scan_workspace(dev, lib.hawk_scan_workspace_bytes(B, T, D, code))
    gws = _gate_workspace(dev, lib.hawk_gate_proj_bwd_weights_workspace_bytes(M, D, nb))
    cws = torch.empty(lib.hawk_conv1d_bwd_workspace_bytes(B, T, D, W), dtype=torch.uint8, device=dev)
    with torch.cuda.device(dev):
        # scan (with the output gate) -> projections' input gradient onto the scan's, in place ->
        # conv -> projections' weight gradients, and one launch for the three closing reductions
        _lib.check("hawk_block_core_bwd", lib.hawk_block_core_bwd(
            xy.data_ptr(), ld, u.data_ptr(), xg.data_ptr(), ag.data_ptr(), h.data_ptr(), conv_w.data_ptr(),
            w_i.data_ptr(), w_a.data_ptr(), _lib.dtype_code(w_i.dtype), lam.data_ptr(), grad_out.data_ptr(),
            d_xy.data_ptr(), D2, du.data_ptr(), dxg.data_ptr(), dag.data_ptr(), dcw.data_ptr(), dcb.data_ptr(),
            dw_i.data_ptr(), db_i.data_ptr(), dw_a.data_ptr(), db_a.data_ptr(), dlam.data_ptr(), B, T, D, nb, W,
            ws.data_ptr(), ws.numel(), gws.data_ptr(), gws.numel(), cws.data_ptr(), cws.numel(),
            _lib.stream_ptr(dev)))
    return d_xy, dcw, dcb, dw_i, db_i, dw_a, db_a, dlam


@torch.library.custom_op("hawk_amd::block_core_fwd", mutates_args=(), device_types="cuda")
def _block_core_fwd_op(
    xy: torch.Tensor, conv_w: torch.Tensor, conv_b: torch.Tensor, w_i: torch.Tensor, b_i: torch.Tensor,
    w_a: torch.Tensor, b_a: torch.Tensor, a_param: torch.Tensor, want_h: bool, want_last: bool,
) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    return _launch_block_core_fwd(xy, conv_w, conv_b, w_i, b_i, w_a, b_a, a_param, want_h, want_last)


@_block_core_fwd_op.register_fake
def _(xy, conv_w, conv_b, w_i, b_i, w_a, b_a, a_param, want_h, want_last):
    B, T, D2 = xy.shape
    D = D2 // 2
    e = lambda *s: torch.empty(s, dtype=torch.bfloat16, device=xy.device)  # noqa: E731
    return (e(B, T, D), e(B, T, D), e(B, T, D), e(B, T, D), e(B, T, D) if want_h else e(0),
            e(B, 1, D) if want_last else e(0))


@torch.library.custom_op("hawk_amd::block_core_bwd", mutates_args=(), device_types="cuda")
def _block_core_bwd_op(
    xy: torch.Tensor, u: torch.Tensor, xg: torch.Tensor, ag: torch.Tensor, h: torch.Tensor, conv_w: torch.Tensor,
    w_i: torch.Tensor, w_a: torch.Tensor, a_param: torch.Tensor, grad_out: torch.Tensor,
) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor,
           torch.Tensor]:
    return _launch_block_core_bwd(xy, u, xg, ag, h, conv_w, w_i, w_a, a_param, grad_out)


@_block_core_bwd_op.register_fake
def _(xy, u, xg, ag, h, conv_w, w_i, w_a, a_param, grad_out):
    nb, bw, _ = w_i.shape
    D = nb * bw
    f = lambda *s: torch.empty(s, dtype=torch.float32, device=xy.device)  # noqa: E731
    return (torch.empty(xy.shape, dtype=torch.bfloat16, device=xy.device), f(conv_w.shape[0], D), f(D),
            f(nb, bw, bw), f(D), f(nb, bw, bw), f(D), f(D))


class BlockCore(Function):
    @staticmethod
    def forward(ctx, xy, conv_w, conv_b, w_i, b_i, w_a, b_a, a_param, want_last):
        from .external import kernel_weights

        assert block_core_layout_ok(xy), "xy must be a [B,T,2D] bf16 tensor the kernels can read in place"
        B, T, D2 = xy.shape
        assert a_param.shape == (D2 // 2,), "Error: a_param does not match the channel count"
        ctx.dtypes = tuple(t.dtype for t in (conv_w, conv_b, w_i, b_i, w_a, b_a, a_param))
        lam = a_param.float().contiguous()
        cw = conv_w.float().contiguous()
        w_i16, w_a16 = kernel_weights(w_i, w_a, B * T)
        want_h = any(ctx.needs_input_grad[:8])
        out, u, xg, ag, h, h_last = _block_core_fwd_op(
            xy, cw, conv_b.float().contiguous(), w_i16, b_i.float().reshape(-1), w_a16, b_a.float().reshape(-1),
            lam, want_h, bool(want_last))
        if want_h:
            ctx.save_for_backward(xy, u, xg, ag, h, cw, w_i16, w_a16, lam)
        ctx.mark_non_differentiable(h_last)
        return out, h_last

    @staticmethod
    def backward(ctx, grad_out, _grad_last):  # type: ignore[override]
        xy, u, xg, ag, h, cw, w_i, w_a, lam = ctx.saved_tensors
        go = grad_out if grad_out.dtype == torch.bfloat16 else grad_out.to(torch.bfloat16)
        go = go if go.is_contiguous() else go.contiguous()
        d_xy, dcw, dcb, dw_i, db_i, dw_a, db_a, dlam = _block_core_bwd_op(xy, u, xg, ag, h, cw, w_i, w_a, lam, go)
        nb, bw, _ = w_i.shape
        t = ctx.dtypes
        return (d_xy, dcw.to(t[0]), dcb.to(t[1]), dw_i.to(t[2]), db_i.reshape(nb, bw).to(t[3]), dw_a.to(t[4]),
                db_a.reshape(nb, bw).to(t[5]), dlam.to(t[6]), None)


def recurrent_block_core(xy, conv, input_gate, a_gate, a_param, return_last_state: bool = False):
    """``gelu(y) * scan(u, input_gate(u), a_gate(u), a_param)`` with ``u = conv(x)`` and
    ``x, y = xy.chunk(2, -1)``, for a bf16 ``xy`` that ``block_core_layout_ok`` accepts and gate
    modules the fused projection kernels serve (``external.gate_projections_supported``)."""
    out, h_last = BlockCore.apply(xy, conv.w, conv.b, input_gate.w, input_gate.b, a_gate.w, a_gate.b, a_param,
                                  return_last_state)
    return (out, h_last) if return_last_state else out
