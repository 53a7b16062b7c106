"""RG-LRU linear scan operator backed by the gfx950 HIP kernels.

Public surface mirrors the upstream operator boundary (hawk/scan_fused.py:319-445):

    sequential_scan_forward(x, x_rg_lru, a_rg_lru, a_param) -> h
    sequential_scan_backward(x, x_rg_lru, a_rg_lru, a_param, h_saved, grad_out)
        -> (dx, dx_rg_lru, da_rg_lru, da_param)
    DiagonalRecurrence            torch.autograd.Function
    fused_linear_scan             = DiagonalRecurrence.apply

Differences from upstream, all deliberate:

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


def _launch_scan_fwd(x, x_rg_lru, a_rg_lru, a_param) -> torch.Tensor:
    dev = _lib.require_cuda(x, x_rg_lru, a_rg_lru, a_param)
    x, x_rg_lru, a_rg_lru, a_param = (_lib.dense16(t) for t in (x, x_rg_lru, a_rg_lru, a_param))
    b, sq, d = x.shape
    code = _lib.dtype_code(x.dtype)
    lib = _lib.load()
    h = torch.empty_like(x)
    nbytes = lib.hawk_scan_workspace_bytes(b, sq, d, code)
    ws = _lib.scan_workspace(dev, nbytes)
    with torch.cuda.device(dev):
        status = lib.hawk_rglru_scan_fwd(
            x.data_ptr(), x_rg_lru.data_ptr(), a_rg_lru.data_ptr(), a_param.data_ptr(), h.data_ptr(),
            b, sq, d, code, ws.data_ptr(), ws.numel(), _lib.stream_ptr(dev),
        )
    _lib.check("hawk_rglru_scan_fwd", status)
    return h


def _launch_scan_bwd(x, x_rg_lru, a_rg_lru, a_param, h_saved, grad_out):
    dev = _lib.require_cuda(x, x_rg_lru, a_rg_lru, a_param, h_saved, grad_out)
    x, x_rg_lru, a_rg_lru, a_param, h_saved, grad_out = (
        _lib.dense16(t) for t in (x, x_rg_lru, a_rg_lru, a_param, h_saved, grad_out)
    )
    b, sq, d = x.shape
    code = _lib.dtype_code(x.dtype)
    lib = _lib.load()
    dx = torch.empty_like(x)
    dxg = torch.empty_like(x)
    dag = torch.empty_like(x)
    dlam = torch.empty(d, dtype=torch.float32, device=dev)
    nbytes = lib.hawk_scan_workspace_bytes(b, sq, d, code)
    ws = _lib.scan_workspace(dev, nbytes)
    with torch.cuda.device(dev):
        status = lib.hawk_rglru_scan_bwd(
            x.data_ptr(), x_rg_lru.data_ptr(), a_rg_lru.data_ptr(), a_param.data_ptr(),
            h_saved.data_ptr(), grad_out.data_ptr(), dx.data_ptr(), dxg.data_ptr(), dag.data_ptr(),
            dlam.data_ptr(), b, sq, d, code, ws.data_ptr(), ws.numel(), _lib.stream_ptr(dev),
        )
    _lib.check("hawk_rglru_scan_bwd", status)
    return dx, dxg, dag, dlam


# ---------------------------------------------------------------------------------------
# torch.library registration (opaque to Dynamo, with shape/dtype propagation rules)
# ---------------------------------------------------------------------------------------
@torch.library.custom_op("hawk_amd::rglru_scan_fwd", mutates_args=(), device_types="cuda")
def _rglru_scan_fwd_op(
    x: torch.Tensor, x_rg_lru: torch.Tensor, a_rg_lru: torch.Tensor, a_param: torch.Tensor
) -> torch.Tensor:
    return _launch_scan_fwd(x, x_rg_lru, a_rg_lru, a_param)


@_rglru_scan_fwd_op.register_fake
def _(x, x_rg_lru, a_rg_lru, a_param):
    return torch.empty_like(x, memory_format=torch.contiguous_format)


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
) -> torch.Tensor:
    """Forward pass of the RG-LRU scan (drop-in for hawk/scan_fused.py:319-360).

    Non-contiguous inputs are silently copied, as upstream does; D must be a multiple of
    64, as upstream asserts.  ``a_param`` is used in fp32 whatever dtype it arrives in.
    """
    _check_shapes(x, x_rg_lru, a_rg_lru, a_param)
    x, x_rg_lru, a_rg_lru = _prepare(x, x_rg_lru, a_rg_lru)
    a_param = a_param.float().contiguous()
    return _rglru_scan_fwd_op(x, x_rg_lru, a_rg_lru, a_param)


def sequential_scan_backward(
    x_saved: torch.Tensor,
    x_rg_lru_saved: torch.Tensor,
    a_rg_lru_saved: torch.Tensor,
    a_param_saved: torch.Tensor,
    h_saved: torch.Tensor,
    grad_out: torch.Tensor,
) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    """Backward pass of the RG-LRU scan (drop-in for hawk/scan_fused.py:363-424).

    Returns (dx, dx_rg_lru, da_rg_lru, da_param[D]); da_param is fp32 and already summed
    over the batch.  A non-contiguous ``grad_out`` is copied with a warning, as upstream.
    """
    _check_shapes(x_saved, x_rg_lru_saved, a_rg_lru_saved, a_param_saved)
    assert h_saved.shape == x_saved.shape and grad_out.shape == x_saved.shape
    if not grad_out.is_contiguous():
        grad_out = grad_out.contiguous()
        warnings.warn(
            "`grad_out` tensor is not contiguous. Setting to contiguous and attempting to continue. "
            "This may impact runtime."
        )
    if grad_out.dtype != x_saved.dtype:
        grad_out = grad_out.to(x_saved.dtype)
    if h_saved.dtype != x_saved.dtype:
        h_saved = h_saved.to(x_saved.dtype)
    x_saved, x_rg_lru_saved, a_rg_lru_saved, h_saved, grad_out = _prepare(
        x_saved, x_rg_lru_saved, a_rg_lru_saved, h_saved, grad_out
    )
    a_param_saved = a_param_saved.float().contiguous()
    return _rglru_scan_bwd_op(x_saved, x_rg_lru_saved, a_rg_lru_saved, a_param_saved, h_saved, grad_out)


def _activation_dtype(x: torch.Tensor) -> torch.dtype:
    """dtype the scan runs in: bf16 under CUDA autocast (as upstream's custom_fwd), else
    bf16 or fp32 as given; other floating dtypes are computed in fp32."""
    if torch.is_autocast_enabled("cuda"):
        return torch.bfloat16
    if x.dtype in (torch.bfloat16, torch.float32):
        return x.dtype
    return torch.float32


class DiagonalRecurrence(Function):
    """h = scan(x, x_rg_lru, a_rg_lru, a_param) with the hand-written reverse-time backward.

    Same four positional tensor arguments and four gradients as upstream
    (hawk/scan_fused.py:426-442).  Under CUDA autocast the three activation tensors are
    cast to bf16, which is what upstream's ``custom_fwd(cast_inputs=torch.bfloat16)`` does
    to them; Lambda is kept in fp32.
    """

    @staticmethod
    def forward(ctx, x, x_rg_lru, a_rg_lru, a_param) -> torch.Tensor:
        run_dtype = _activation_dtype(x)
        out_dtype = run_dtype if run_dtype == torch.bfloat16 or x.dtype == torch.float32 else x.dtype
        xc, xgc, agc = (t.to(run_dtype) for t in (x, x_rg_lru, a_rg_lru))
        h = sequential_scan_forward(xc, xgc, agc, a_param)
        ctx.save_for_backward(xc, xgc, agc, a_param, h)
        return h if h.dtype == out_dtype else h.to(out_dtype)

    @staticmethod
    def backward(ctx, grad_output):  # type: ignore[override]
        (x, x_rg_lru, a_rg_lru, a_param, h_saved) = ctx.saved_tensors
        x_grad, x_rg_lru_grad, a_rg_lru_grad, a_param_grad = sequential_scan_backward(
            x, x_rg_lru, a_rg_lru, a_param, h_saved, grad_output
        )
        return x_grad, x_rg_lru_grad, a_rg_lru_grad, a_param_grad.to(a_param.dtype)


fused_linear_scan = DiagonalRecurrence.apply
