"""Building blocks around the scan: the temporal Conv1D (HIP kernels), the block-diagonal
gate projection and the Lambda initialiser.

``Conv1D`` keeps the module surface of upstream's hawk/external.py:12-98 (constructor
arguments, parameter names ``w`` [temporal_width, width] and ``b`` [width], fp32) but its
forward and backward are single streaming HIP kernels instead of a Python loop of
slice / pad / concat / multiply passes differentiated by autograd.
"""

from __future__ import annotations

import math
from typing import Optional, Tuple

import torch
import torch.nn as nn
from torch.autograd import Function

from . import _lib

MAX_TEMPORAL_WIDTH = 8


# ---------------------------------------------------------------------------------------
# conv1d custom ops
# ---------------------------------------------------------------------------------------
def _launch_conv_fwd(x, w, b, state, out_dtype) -> torch.Tensor:
    tensors = [x, w, b] + ([state] if state is not None else [])
    dev = _lib.require_cuda(*tensors)
    x, w, b = _lib.dense16(x), _lib.dense16(w), _lib.dense16(b)
    if state is not None:
        state = _lib.dense16(state)
    B, T, D = x.shape
    W = w.shape[0]
    y = _lib.activation_empty((B, T, D), out_dtype, dev)
    lib = _lib.load()
    with torch.cuda.device(dev):
        status = lib.hawk_conv1d_fwd(
            x.data_ptr(), w.data_ptr(), b.data_ptr(), _lib.ptr(state), y.data_ptr(),
            B, T, D, W, _lib.dtype_code(x.dtype), _lib.dtype_code(out_dtype), _lib.stream_ptr(dev),
        )
    _lib.check("hawk_conv1d_fwd", status)
    return y


def _launch_conv_bwd(grad_y, x, w):
    dev = _lib.require_cuda(grad_y, x, w)
    grad_y, x, w = _lib.dense16(grad_y), _lib.dense16(x), _lib.dense16(w)
    B, T, D = x.shape
    W = w.shape[0]
    dx = _lib.activation_empty(x.shape, x.dtype, dev)
    dw = torch.empty((W, D), dtype=torch.float32, device=dev)
    db = torch.empty((D,), dtype=torch.float32, device=dev)
    lib = _lib.load()
    nbytes = lib.hawk_conv1d_bwd_workspace_bytes(B, T, D, W)
    ws = torch.empty(nbytes, dtype=torch.uint8, device=dev)
    with torch.cuda.device(dev):
        status = lib.hawk_conv1d_bwd(
            grad_y.data_ptr(), x.data_ptr(), w.data_ptr(), dx.data_ptr(), dw.data_ptr(), db.data_ptr(),
            B, T, D, W, _lib.dtype_code(x.dtype), _lib.dtype_code(grad_y.dtype),
            ws.data_ptr(), ws.numel(), _lib.stream_ptr(dev),
        )
    _lib.check("hawk_conv1d_bwd", status)
    return dx, dw, db


@torch.library.custom_op("hawk_amd::conv1d_fwd", mutates_args=(), device_types="cuda")
def _conv1d_fwd_op(
    x: torch.Tensor, w: torch.Tensor, b: torch.Tensor, state: Optional[torch.Tensor], out_fp32: bool
) -> torch.Tensor:
    return _launch_conv_fwd(x, w, b, state, torch.float32 if out_fp32 else torch.bfloat16)


@_conv1d_fwd_op.register_fake
def _(x, w, b, state, out_fp32):
    return torch.empty(x.shape, dtype=torch.float32 if out_fp32 else torch.bfloat16, device=x.device)


@torch.library.custom_op("hawk_amd::conv1d_bwd", mutates_args=(), device_types="cuda")
def _conv1d_bwd_op(
    grad_y: torch.Tensor, x: torch.Tensor, w: torch.Tensor
) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    return _launch_conv_bwd(grad_y, x, w)


@_conv1d_bwd_op.register_fake
def _(grad_y, x, w):
    return (
        torch.empty_like(x, memory_format=torch.contiguous_format),
        torch.empty(w.shape, dtype=torch.float32, device=x.device),
        torch.empty((x.shape[-1],), dtype=torch.float32, device=x.device),
    )


class _TemporalConv(Function):
    """y = causal depthwise conv(x; w, b) with zero history; hand-written backward."""

    @staticmethod
    def forward(ctx, x, w, b, out_fp32: bool):
        xc = x if x.is_contiguous() else x.contiguous()
        ctx.save_for_backward(xc, w)
        ctx.in_dtype = x.dtype
        return _conv1d_fwd_op(xc, w, b, None, out_fp32)

    @staticmethod
    def backward(ctx, grad_y):  # type: ignore[override]
        xc, w = ctx.saved_tensors
        if grad_y.dtype not in (torch.bfloat16, torch.float32):
            grad_y = grad_y.float()
        gy = grad_y if grad_y.is_contiguous() else grad_y.contiguous()
        dx, dw, db = _conv1d_bwd_op(gy, xc, w)
        return dx, dw, db, None


def temporal_conv1d(x, w, b, out_dtype: Optional[torch.dtype] = None, state=None):
    """Functional form: x [B,T,D] (bf16 or fp32), w [W,D] fp32, b [D] fp32.

    ``out_dtype`` defaults to the promotion of x and w dtypes (fp32), which is what
    upstream's ``x_window * w`` produces (hawk/external.py:90).  With ``state``
    ([B,W-1,D], the rows preceding x) no gradient is defined.
    """
    assert x.dim() == 3, f"expected x of shape [B,T,D], got {tuple(x.shape)}"
    W, D = w.shape
    assert x.shape[-1] == D and b.shape == (D,), "conv weight / bias do not match the channel count"
    assert 1 <= W <= MAX_TEMPORAL_WIDTH, f"temporal width must be in [1, {MAX_TEMPORAL_WIDTH}]"
    if x.dtype not in (torch.bfloat16, torch.float32):
        x = x.float()
    if out_dtype is None:
        out_dtype = torch.promote_types(x.dtype, w.dtype)
    assert out_dtype in (torch.bfloat16, torch.float32)
    w32, b32 = w.float(), b.float()
    if state is not None:
        assert state.shape == (x.shape[0], W - 1, D)
        xc = x if x.is_contiguous() else x.contiguous()
        return _conv1d_fwd_op(xc, w32, b32, state.to(x.dtype), out_dtype == torch.float32)
    return _TemporalConv.apply(x, w32, b32, out_dtype == torch.float32)


class Conv1D(nn.Module):
    """Causal depthwise temporal convolution, y_t = b + sum_s w[W-1-s] * x_{t-s}.

    Drop-in for upstream's ``Conv1D(width, temporal_width)`` (hawk/external.py:12-47):
    same parameters (``w`` drawn from N(0, w_init_variance_scale / temporal_width), ``b``
    zero) and ``forward(x) -> y``.  ``out_dtype=None`` reproduces upstream's type
    promotion (fp32 output for bf16 input); pass ``torch.bfloat16`` to keep activations
    in bf16 and halve the write traffic.
    """

    def __init__(
        self,
        width: int,
        temporal_width: int,
        w_init_variance_scale: float = 0.01,
        out_dtype: Optional[torch.dtype] = None,
    ):
        super().__init__()
        self.width = width
        self.temporal_width = temporal_width
        self.w_init_variance_scale = w_init_variance_scale
        self.out_dtype = out_dtype
        self.w = nn.Parameter(torch.empty([temporal_width, width], dtype=torch.float32))
        self.b = nn.Parameter(torch.empty([width], dtype=torch.float32))
        self.reset_parameters()

    def reset_parameters(self) -> None:
        nn.init.normal_(self.w, mean=0.0, std=math.sqrt(self.w_init_variance_scale / self.temporal_width))
        nn.init.zeros_(self.b)

    def forward(self, x: torch.Tensor, state: Optional[torch.Tensor] = None) -> torch.Tensor:
        return temporal_conv1d(x, self.w, self.b, self.out_dtype, state)

    def step(self, conv_state: torch.Tensor, x_new: torch.Tensor) -> torch.Tensor:
        """Decode step: rolls ``conv_state`` [B,W-1,D] in place and returns y [B,1,D]."""
        return temporal_conv1d_step(conv_state, x_new, self.w, self.b, self.out_dtype)


def temporal_conv1d_step(conv_state, x_new, w, b, out_dtype: Optional[torch.dtype] = None):
    """One-token conv: window = concat(conv_state, x_new); conv_state is updated in place
    (rolled up one row, x_new written last).  Replaces hawk/hawk.py:169-179 +
    hawk/cache.py:37-43 upstream.  x_new is [B,1,D] or [B,D]; returns the same rank."""
    W, D = w.shape
    squeeze = x_new.dim() == 2
    xn = x_new.reshape(x_new.shape[0], D)
    B = xn.shape[0]
    assert conv_state.shape == (B, W - 1, D), (
        f"conv_state must be [B, W-1, D] = {(B, W - 1, D)}, got {tuple(conv_state.shape)}"
    )
    assert conv_state.is_contiguous(), "conv_state is updated in place and must be contiguous"
    dev = _lib.require_cuda(conv_state, xn, w, b)
    xn = _lib.dense16(xn.to(conv_state.dtype))
    if out_dtype is None:
        out_dtype = torch.promote_types(conv_state.dtype, w.dtype)
    y = torch.empty((B, D), dtype=out_dtype, device=dev)
    w32, b32 = _lib.dense16(w.detach().float()), _lib.dense16(b.detach().float())
    with torch.cuda.device(dev):
        status = _lib.load().hawk_conv1d_step(
            conv_state.data_ptr(), xn.data_ptr(), w32.data_ptr(), b32.data_ptr(), y.data_ptr(),
            B, D, W, _lib.dtype_code(conv_state.dtype), _lib.dtype_code(out_dtype), _lib.stream_ptr(dev),
        )
    _lib.check("hawk_conv1d_step", status)
    return y if squeeze else y.unsqueeze(1)


def rglru_step(x, x_rg_lru, a_rg_lru, a_param, recc_state):
    """One-token RG-LRU update.  ``recc_state`` [B,1,D] or [B,D] is read and overwritten
    with the new state; the new state is also returned in x's dtype and shape.
    Replaces Hawk.inference_prologue + step + cache write (hawk/hawk.py:137-151, :196-198)."""
    D = x.shape[-1]
    shape = x.shape
    B = x.numel() // D
    assert recc_state.numel() == B * D and recc_state.is_contiguous()
    dev = _lib.require_cuda(x, x_rg_lru, a_rg_lru, a_param, recc_state)
    run_dtype = x.dtype if x.dtype in (torch.bfloat16, torch.float32) else torch.float32
    xs = [_lib.dense16(t.reshape(B, D).to(run_dtype)) for t in (x, x_rg_lru, a_rg_lru)]
    lam = _lib.dense16(a_param.detach().float())
    h = torch.empty((B, D), dtype=run_dtype, device=dev)
    with torch.cuda.device(dev):
        status = _lib.load().hawk_rglru_step(
            xs[0].data_ptr(), xs[1].data_ptr(), xs[2].data_ptr(), lam.data_ptr(),
            recc_state.data_ptr(), h.data_ptr(), B, D,
            _lib.dtype_code(run_dtype), _lib.dtype_code(recc_state.dtype), _lib.stream_ptr(dev),
        )
    _lib.check("hawk_rglru_step", status)
    return h.reshape(shape)


def rglru_step_gated(x, x_rg_lru, a_rg_lru, a_param, recc_state, y, bias_i=None, bias_a=None):
    """One-token RG-LRU update fused with what surrounds it in a Hawk block: the two gate
    projections' biases (``bias_i``, ``bias_a``, any shape with D elements, optional) are
    added to the logits in the kernel, the state is updated in place and
    ``gelu(y) * h`` is returned (hawk/hawk.py:134-151, :181-182, :196-198 in one launch).
    ``y`` may be a slice of a wider tensor (the gate half of the input projection)."""
    D = x.shape[-1]
    shape = x.shape
    B = x.numel() // D
    assert recc_state.numel() == B * D and recc_state.is_contiguous()
    dev = _lib.require_cuda(x, x_rg_lru, a_rg_lru, a_param, recc_state, y)
    run_dtype = x.dtype if x.dtype in (torch.bfloat16, torch.float32) else torch.float32
    xs = [_lib.dense16(t.reshape(B, D).to(run_dtype)) for t in (x, x_rg_lru, a_rg_lru)]
    lam = _lib.dense16(a_param.detach().float())
    biases = [None if b is None else _lib.dense16(b.detach().float().reshape(D)) for b in (bias_i, bias_a)]
    y2 = y.reshape(B, D) if y.dtype == run_dtype else y.reshape(B, D).to(run_dtype)
    if y2.stride(1) != 1 or (B > 1 and y2.stride(0) < D):
        y2 = y2.contiguous()
    ldy = y2.stride(0) if B > 1 else D
    out = torch.empty((B, D), dtype=run_dtype, device=dev)
    with torch.cuda.device(dev):
        status = _lib.load().hawk_rglru_step_gated(
            xs[0].data_ptr(), xs[1].data_ptr(), xs[2].data_ptr(), _lib.ptr(biases[0]), _lib.ptr(biases[1]),
            lam.data_ptr(), y2.data_ptr(), ldy, recc_state.data_ptr(), None, out.data_ptr(), B, D,
            _lib.dtype_code(run_dtype), _lib.dtype_code(recc_state.dtype), _lib.stream_ptr(dev),
        )
    _lib.check("hawk_rglru_step_gated", status)
    return out.reshape(shape)


def decode_core_supported(x_new: torch.Tensor, conv: "Conv1D", gate: "BlockDiagonalLinear",
                          conv_state: torch.Tensor) -> bool:
    """Whether ``decode_core_step`` serves these operands: bf16 activations and conv window, a
    block width of 32..256 (the fused projections' rule) and a window of at most 8 rows."""
    if x_new.device.type != "cuda" or x_new.dtype != torch.bfloat16 or conv_state.dtype != torch.bfloat16:
        return False
    if gate.w.dtype not in (torch.bfloat16, torch.float32):
        return False
    W = conv.w.shape[0]
    return (1 <= W <= MAX_TEMPORAL_WIDTH and gate.width % gate.num_blocks == 0
            and gate.block_width in _GATE_BLOCK_WIDTHS)


def decode_core_step(conv_state, x_new, conv: "Conv1D", input_gate: "BlockDiagonalLinear",
                     a_gate: "BlockDiagonalLinear", a_param, recc_state, y):
    """One decode step of a Hawk block's recurrent core in one launch.

    ``conv_state`` [B, W-1, D] is rolled in place and ``recc_state`` [B, 1, D] or [B, D] is
    overwritten with the new state; returns ``gelu(y) * h`` in x_new's shape.  Same result
    (to the last bit or two of bf16) as ``temporal_conv1d_step`` + ``gate_projections`` +
    ``rglru_step_gated``; upstream: hawk/hawk.py:134-151, :169-182, :196-198 and
    hawk/cache.py:29-43.  ``x_new`` and ``y`` may be the two halves of the input projection,
    passed in place.
    """
    W, D = conv.w.shape
    shape = x_new.shape
    B = x_new.numel() // D
    assert conv_state.shape == (B, W - 1, D) and conv_state.is_contiguous(), (
        f"conv_state must be a contiguous [B, W-1, D] = {(B, W - 1, D)}, got {tuple(conv_state.shape)}"
    )
    assert recc_state.numel() == B * D and recc_state.is_contiguous()
    assert x_new.dtype == torch.bfloat16 and conv_state.dtype == torch.bfloat16, "the fused step runs on bf16"
    dev = _lib.require_cuda(conv_state, x_new, conv.w, input_gate.w, a_gate.w, a_param, recc_state, y)

    def rows(t):
        """[B, D] view with unit column stride and its row stride, copying only if it must."""
        t2 = t.reshape(B, D) if t.dtype == torch.bfloat16 else t.reshape(B, D).to(torch.bfloat16)
        if t2.stride(1) != 1 or (B > 1 and t2.stride(0) < D):
            t2 = t2.contiguous()
        return t2, (t2.stride(0) if B > 1 else D)

    xn, ldx = rows(x_new)
    if ldx % 8 != 0 or xn.data_ptr() % 16 != 0:
        xn, ldx = _lib.dense16(xn.contiguous()), D
    y2, ldy = rows(y)
    w32, b32 = _lib.dense16(conv.w.detach().float()), _lib.dense16(conv.b.detach().float())
    w_i, w_a = _lib.dense16(input_gate.w.detach()), _lib.dense16(a_gate.w.detach())
    if w_a.dtype != w_i.dtype:
        w_a = w_a.to(w_i.dtype)
    b_i = _lib.dense16(input_gate.b.detach().float().reshape(D))
    b_a = _lib.dense16(a_gate.b.detach().float().reshape(D))
    lam = _lib.dense16(a_param.detach().float())
    out = torch.empty((B, D), dtype=torch.bfloat16, device=dev)
    lib = _lib.load()
    with torch.cuda.device(dev):
        # counters that let several workgroups share a block's output columns
        nws = lib.hawk_decode_core_workspace_bytes(B, D, input_gate.num_blocks)
        ws = _lib.decode_workspace(dev, nws)
        status = lib.hawk_decode_core_step_ws(
            conv_state.data_ptr(), xn.data_ptr(), ldx, w32.data_ptr(), b32.data_ptr(), w_i.data_ptr(),
            b_i.data_ptr(), w_a.data_ptr(), b_a.data_ptr(), lam.data_ptr(), y2.data_ptr(), ldy,
            recc_state.data_ptr(), out.data_ptr(), B, D, input_gate.num_blocks, W, _lib.HAWK_DTYPE_BF16,
            _lib.dtype_code(w_i.dtype), _lib.dtype_code(recc_state.dtype), ws.data_ptr(), ws.numel(),
            _lib.stream_ptr(dev),
        )
    _lib.check("hawk_decode_core_step_ws", status)
    return out.reshape(shape)


# ---------------------------------------------------------------------------------------
# Pieces of the harness model that are not on the hot path (library GEMMs, initialisers).
# ---------------------------------------------------------------------------------------
def rnn_param_init(
    tensor: torch.Tensor, min_rad: float, max_rad: float, transform: str = "softplus", eps: float = 1e-8
) -> torch.Tensor:
    """Draws Lambda so that exp(-softplus(Lambda))^2 is uniform in [min_rad^2, max_rad^2]
    (same distribution as hawk/external.py:153-168 upstream)."""
    if transform != "softplus":
        raise NotImplementedError(f"transform {transform!r}")
    with torch.no_grad():
        u = torch.empty_like(tensor).uniform_(min_rad**2 + eps, max_rad**2 + eps)
        # softplus(L) = -0.5 ln(u)  <=>  L = ln(u^(-1/2) - 1)
        tensor.copy_(torch.log(torch.expm1(-0.5 * torch.log(u))))
    return tensor


class BlockDiagonalLinear(nn.Module):
    """y = blockdiag(w_0..w_{n-1}) x + b: the gate projections of the RG-LRU.

    Parameter names and shapes follow hawk/external.py:200-209 upstream (``w``
    [num_blocks, block_width, block_width], ``b`` [num_blocks, block_width]).  The
    contraction is a batched library GEMM (rocBLAS through torch.bmm-style einsum); it is
    dense MFMA work and not part of the memory-bound scan path.
    """

    def __init__(self, width: int, num_blocks: int, w_init_variance_scale: float = 1.0, device=None, dtype=None):
        super().__init__()
        assert width % num_blocks == 0, "width must be divisible by num_blocks"
        self.width = width
        self.num_blocks = num_blocks
        self.w_init_variance_scale = w_init_variance_scale
        self.block_width = width // num_blocks
        shape = (num_blocks, self.block_width, self.block_width)
        self.w = nn.Parameter(torch.empty(shape, device=device, dtype=dtype))
        self.b = nn.Parameter(torch.empty(shape[:2], device=device, dtype=dtype))
        self.reset_parameters()

    def reset_parameters(self) -> None:
        nn.init.normal_(self.w, mean=0.0, std=math.sqrt(self.w_init_variance_scale / self.block_width))
        nn.init.zeros_(self.b)

    def forward(self, x: torch.Tensor, add_bias: bool = True) -> torch.Tensor:
        """``add_bias=False`` leaves ``b`` out for a consumer that adds it itself (the fused
        decode step does)."""
        lead = x.shape[:-1]
        xb = x.reshape(*lead, self.num_blocks, self.block_width)
        yb = torch.einsum("...hi,hij->...hj", xb, self.w)
        if add_bias:
            yb = yb + self.b
        return yb.reshape(*lead, self.width)


# ---------------------------------------------------------------------------------------
# Both gate projections in one pass (matrix-core kernels): the pair of BlockDiagonalLinear
# calls of hawk/hawk.py:181-182 and their autograd.
# ---------------------------------------------------------------------------------------
_gate_ws: dict = {}
_GATE_BLOCK_WIDTHS = (32, 64, 128, 256)


def _gate_workspace(dev: torch.device, nbytes: int) -> torch.Tensor:
    if torch.cuda.is_current_stream_capturing():
        return torch.empty(nbytes, dtype=torch.uint8, device=dev)  # the graph's own scratch, from its pool
    key = (dev.index if dev.index is not None else torch.cuda.current_device(), _lib.stream_ptr(dev))
    with _lib._lock:
        ws = _gate_ws.get(key)
        if ws is None or ws.numel() < nbytes:
            ws = torch.empty(nbytes, dtype=torch.uint8, device=dev)
            _gate_ws[key] = ws
    return ws


def _launch_gate_fwd(x, w_i, b_i, w_a, b_a, out_bf16: bool):
    dev = _lib.require_cuda(x, w_i, b_i, w_a, b_a)
    nb, bw, _ = w_i.shape
    D = nb * bw
    M = x.numel() // D
    x2, w_i, w_a, b_i, b_a = (_lib.dense16(t) for t in (x.reshape(M, D), w_i, w_a, b_i, b_a))
    out_dtype = torch.bfloat16 if out_bf16 else torch.float32
    xg = _lib.activation_empty(x.shape, out_dtype, dev)
    ag = _lib.activation_empty(x.shape, out_dtype, dev)
    with torch.cuda.device(dev):
        status = _lib.load().hawk_gate_proj_fwd(
            x2.data_ptr(), w_i.data_ptr(), b_i.data_ptr(), w_a.data_ptr(), b_a.data_ptr(), xg.data_ptr(),
            ag.data_ptr(), M, D, nb, _lib.dtype_code(x2.dtype), _lib.dtype_code(w_i.dtype),
            _lib.dtype_code(out_dtype), _lib.stream_ptr(dev),
        )
    _lib.check("hawk_gate_proj_fwd", status)
    return xg, ag


def _launch_gate_bwd(x, d_xg, d_ag, w_i, w_a, addend=None):
    dev = _lib.require_cuda(x, d_xg, d_ag, w_i, w_a)
    nb, bw, _ = w_i.shape
    D = nb * bw
    M = x.numel() // D
    x2, g_i, g_a, w_i, w_a = (_lib.dense16(t) for t in (x.reshape(M, D), d_xg.reshape(M, D), d_ag.reshape(M, D), w_i, w_a))
    lib = _lib.load()
    dx = _lib.activation_empty(x.shape, x.dtype, dev)
    if addend is not None:
        addend = _lib.dense16(addend.reshape(M, D).to(x.dtype))
    dw_i = torch.empty((nb, bw, bw), dtype=torch.float32, device=dev)
    dw_a = torch.empty_like(dw_i)
    db_i = torch.empty(D, dtype=torch.float32, device=dev)
    db_a = torch.empty(D, dtype=torch.float32, device=dev)
    nbytes = lib.hawk_gate_proj_bwd_weights_workspace_bytes(M, D, nb)
    ws = _gate_workspace(dev, nbytes)
    with torch.cuda.device(dev):
        st = _lib.stream_ptr(dev)
        status = lib.hawk_gate_proj_bwd_input(
            g_i.data_ptr(), g_a.data_ptr(), w_i.data_ptr(), w_a.data_ptr(), _lib.ptr(addend), dx.data_ptr(), M, D, nb,
            _lib.dtype_code(g_i.dtype), _lib.dtype_code(w_i.dtype), _lib.dtype_code(dx.dtype), st,
        )
        _lib.check("hawk_gate_proj_bwd_input", status)
        status = lib.hawk_gate_proj_bwd_weights(
            x2.data_ptr(), g_i.data_ptr(), g_a.data_ptr(), dw_i.data_ptr(), db_i.data_ptr(), dw_a.data_ptr(),
            db_a.data_ptr(), M, D, nb, _lib.dtype_code(x2.dtype), _lib.dtype_code(g_i.dtype), ws.data_ptr(),
            ws.numel(), st,
        )
        _lib.check("hawk_gate_proj_bwd_weights", status)
    return dx, dw_i, db_i, dw_a, db_a


@torch.library.custom_op("hawk_amd::gate_proj_fwd", mutates_args=(), device_types="cuda")
def _gate_proj_fwd_op(
    x: torch.Tensor, w_i: torch.Tensor, b_i: torch.Tensor, w_a: torch.Tensor, b_a: torch.Tensor, out_bf16: bool
) -> Tuple[torch.Tensor, torch.Tensor]:
    return _launch_gate_fwd(x, w_i, b_i, w_a, b_a, out_bf16)


@_gate_proj_fwd_op.register_fake
def _(x, w_i, b_i, w_a, b_a, out_bf16):
    dt = torch.bfloat16 if out_bf16 else torch.float32
    return torch.empty(x.shape, dtype=dt, device=x.device), torch.empty(x.shape, dtype=dt, device=x.device)


@torch.library.custom_op("hawk_amd::gate_proj_bwd", mutates_args=(), device_types="cuda")
def _gate_proj_bwd_op(
    x: torch.Tensor, d_xg: torch.Tensor, d_ag: torch.Tensor, w_i: torch.Tensor, w_a: torch.Tensor,
    addend: Optional[torch.Tensor] = None,
) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    return _launch_gate_bwd(x, d_xg, d_ag, w_i, w_a, addend)


@_gate_proj_bwd_op.register_fake
def _(x, d_xg, d_ag, w_i, w_a, addend=None):
    nb, bw, _ = w_i.shape
    f32 = dict(dtype=torch.float32, device=x.device)
    return (
        torch.empty(x.shape, dtype=x.dtype, device=x.device),
        torch.empty((nb, bw, bw), **f32), torch.empty(nb * bw, **f32),
        torch.empty((nb, bw, bw), **f32), torch.empty(nb * bw, **f32),
    )


# The projection kernels round fp32 weights to bf16 as they load them, every workgroup for
# itself, and moving 512 KiB instead of 256 KiB per workgroup through its L1 makes the forward
# 8 us and the input gradient 13 us longer at a block width of 256.  From this many rows on,
# where the GPU and not the host sets the pace, the weights are rounded once per forward instead
# (the same rounding, so the same results) and the bf16 copies serve the backward too.
_CAST_WEIGHTS_MIN_ROWS = 8192


def kernel_weights(w_i: torch.Tensor, w_a: torch.Tensor, rows: int):
    if w_i.dtype == torch.float32 and rows >= _CAST_WEIGHTS_MIN_ROWS:
        nb, bw, _ = w_i.shape
        if w_i.is_cuda and w_a.dtype == torch.float32 and w_a.shape == w_i.shape and bw % 4 == 0:
            # both gates in one launch
            wi, wa = _lib.dense16(w_i.detach()), _lib.dense16(w_a.detach())
            both = torch.empty((2, nb, bw, bw), dtype=torch.bfloat16, device=w_i.device)
            with torch.cuda.device(w_i.device):
                _lib.check("hawk_gate_weights_to_bf16", _lib.load().hawk_gate_weights_to_bf16(
                    wi.data_ptr(), wa.data_ptr(), both[0].data_ptr(), both[1].data_ptr(), nb, bw,
                    _lib.stream_ptr(w_i.device)))
            return both[0], both[1]
        return w_i.detach().to(torch.bfloat16), w_a.detach().to(torch.bfloat16)
    return w_i, w_a


class _GateProjection(Function):
    """(x_rg_lru, a_rg_lru) = (blockdiag(w_i) x + b_i, blockdiag(w_a) x + b_a), bf16 operands."""

    @staticmethod
    def forward(ctx, x, w_i, b_i, w_a, b_a, out_bf16: bool):
        xc = x if x.is_contiguous() else x.contiguous()
        ctx.param_dtypes = (w_i.dtype, b_i.dtype, w_a.dtype, b_a.dtype)
        w_i, w_a = kernel_weights(w_i, w_a, xc.numel() // xc.shape[-1])
        ctx.save_for_backward(xc, w_i, w_a)
        return _gate_proj_fwd_op(xc, w_i, b_i.float().reshape(-1), w_a, b_a.float().reshape(-1), out_bf16)

    @staticmethod
    def backward(ctx, d_xg, d_ag):  # type: ignore[override]
        x, w_i, w_a = ctx.saved_tensors
        gdt = torch.bfloat16 if (d_xg.dtype == torch.bfloat16 and d_ag.dtype == torch.bfloat16) else torch.float32
        d_xg, d_ag = (g.to(gdt).contiguous() for g in (d_xg, d_ag))
        dx, dw_i, db_i, dw_a, db_a = _gate_proj_bwd_op(x, d_xg, d_ag, w_i, w_a)
        nb, bw, _ = w_i.shape
        dts = ctx.param_dtypes
        return (dx, dw_i.to(dts[0]), db_i.reshape(nb, bw).to(dts[1]), dw_a.to(dts[2]),
                db_a.reshape(nb, bw).to(dts[3]), None)


def gate_projections_supported(x: torch.Tensor, gate: "BlockDiagonalLinear") -> bool:
    """The fused kernels compute with bf16 operands, which is the arithmetic of this einsum
    under bf16 autocast or on bf16 tensors; plain fp32 calls keep the library GEMM."""
    if x.device.type != "cuda" or x.dtype not in (torch.bfloat16, torch.float32):
        return False
    if gate.w.dtype not in (torch.bfloat16, torch.float32):
        return False
    if not (x.dtype == torch.bfloat16 or torch.is_autocast_enabled("cuda")):
        return False
    # same rule as hawk_gate_proj_supported(), restated so that a tracing compiler sees plain Python
    return gate.width % gate.num_blocks == 0 and gate.block_width in _GATE_BLOCK_WIDTHS


def gate_projections(x: torch.Tensor, input_gate: "BlockDiagonalLinear", a_gate: "BlockDiagonalLinear",
                     out_dtype: Optional[torch.dtype] = None) -> Tuple[torch.Tensor, torch.Tensor]:
    """Both gate logits of hawk/hawk.py:181-182, ``(input_gate(x), a_gate(x))``.

    One kernel reads x once and writes both logits (and one pair of kernels does the whole
    backward) whenever ``gate_projections_supported``; otherwise the two modules are called
    as upstream does.  ``out_dtype`` (bf16 or fp32) applies to the fused path and defaults to
    x's dtype.
    """
    if not gate_projections_supported(x, input_gate):
        return input_gate(x), a_gate(x)
    assert a_gate.width == input_gate.width and a_gate.num_blocks == input_gate.num_blocks
    out_bf16 = (out_dtype or x.dtype) == torch.bfloat16
    return _GateProjection.apply(x, input_gate.w, input_gate.b, a_gate.w, a_gate.b, out_bf16)
