"""TEST INFRASTRUCTURE, NOT PRODUCT CODE.

A second, independent CPU statement of the RG-LRU recurrence: a Python loop over time of
the one-token decode arithmetic (hawk/hawk.py:137-151 and :196 upstream), differentiated by
torch.autograd.  It exists for two reasons:

* it derives the gradients by automatic differentiation, so agreement with the analytic
  backward formulas of the C oracle pins both;
* it is the "PyTorch CPU scan" timed as the cpu_baseline of bench.py (upstream has no
  CPU implementation of the full-sequence scan; this loop is the closest thing to one).

The square root uses the same bounded derivative as hawk/scan_fused.py:10-15 upstream
(1/sqrt(max(4z, 1e-6))), so the clip is part of what autograd sees.
"""

from __future__ import annotations

import torch
import torch.nn.functional as F

_MAX_SQRT_GRADIENT = 1000.0


class _BoundedSqrt(torch.autograd.Function):
    """sqrt(z) whose derivative is capped at _MAX_SQRT_GRADIENT."""

    @staticmethod
    def forward(ctx, z):
        ctx.save_for_backward(z)
        return torch.sqrt(z)

    @staticmethod
    def backward(ctx, grad):
        (z,) = ctx.saved_tensors
        floor = 1.0 / (_MAX_SQRT_GRADIENT * _MAX_SQRT_GRADIENT)
        return grad / torch.sqrt(torch.clamp(4.0 * z, min=floor))


def rglru_step(x_t, xg_t, ag_t, a_param, h_prev):
    """One step: returns h_t.  All of x_t, xg_t, ag_t, h_prev are [B, D]."""
    gate_x = torch.sigmoid(xg_t)
    gate_a = torch.sigmoid(ag_t)
    log_a = -8.0 * gate_a * F.softplus(a_param)
    a = torch.exp(log_a)
    mult = _BoundedSqrt.apply(1.0 - torch.exp(2.0 * log_a))
    return a * h_prev + (x_t * gate_x) * mult


def rglru_scan_loop(x, x_rg_lru, a_rg_lru, a_param):
    """h[B,T,D] by looping rglru_step over time from h = 0."""
    B, T, D = x.shape
    h_prev = torch.zeros(B, D, dtype=x.dtype, device=x.device)
    rows = []
    for t in range(T):
        h_prev = rglru_step(x[:, t], x_rg_lru[:, t], a_rg_lru[:, t], a_param, h_prev)
        rows.append(h_prev)
    return torch.stack(rows, dim=1)


def rglru_scan_fwd_bwd(x, x_rg_lru, a_rg_lru, a_param, grad_out):
    """Forward plus autograd backward.  Returns (h, dx, dx_rg_lru, da_rg_lru, dLambda)."""
    leaves = [v.detach().clone().requires_grad_(True) for v in (x, x_rg_lru, a_rg_lru, a_param)]
    h = rglru_scan_loop(*leaves)
    grads = torch.autograd.grad(h, leaves, grad_out)
    return (h.detach(), *grads)


def conv1d_library(x, w, b):
    """Depthwise causal conv through the library routine F.conv1d (left pad W-1)."""
    W, D = w.shape
    T = x.shape[1]
    y = F.conv1d(
        x.transpose(1, 2), w.t().unsqueeze(1).contiguous(), b, padding=W - 1, groups=D
    )[..., :T]
    return y.transpose(1, 2)
