"""TEST INFRASTRUCTURE, NOT PRODUCT CODE.

numpy front end of the C oracle in ``rglru_oracle.c`` (fp64 ground truth and a scalar fp32
port of the same loops).  Only ``tests/``, ``__graft_entry__.smoke()`` and the
``cpu_baseline`` leg of ``bench.py`` may import this package.

Every function here takes and returns numpy arrays; nothing touches a GPU.
"""

from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "_build", "librglru_oracle.so")
_lib = None


def build(force: bool = False) -> str:
    """Compile the C oracle with gcc (``make`` in this directory)."""
    if force:
        subprocess.run(["make", "-C", _HERE, "clean"], check=True, capture_output=True)
    subprocess.run(["make", "-C", _HERE], check=True, capture_output=True)
    return _LIB_PATH


def _load():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = ctypes.CDLL(_LIB_PATH)
    return _lib


def _np_dtype(precision: str):
    if precision == "f64":
        return np.float64
    if precision == "f32":
        return np.float32
    raise ValueError(f"precision must be 'f64' or 'f32', got {precision!r}")


def _prep(a, dt):
    return np.ascontiguousarray(np.asarray(a), dtype=dt)


def _ptr(a):
    return a.ctypes.data_as(ctypes.c_void_p) if a is not None else None


def rglru_scan_fwd(x, x_rg_lru, a_rg_lru, a_param, precision: str = "f64"):
    """h[B,T,D] of the RG-LRU scan (restates hawk/scan_fused.py:44-109)."""
    dt = _np_dtype(precision)
    x, xg, ag, lam = (_prep(v, dt) for v in (x, x_rg_lru, a_rg_lru, a_param))
    B, T, D = x.shape
    assert xg.shape == x.shape and ag.shape == x.shape and lam.shape == (D,)
    h = np.empty_like(x)
    fn = getattr(_load(), f"oracle_rglru_scan_fwd_{precision}")
    fn(_ptr(x), _ptr(xg), _ptr(ag), _ptr(lam), _ptr(h), B, T, D)
    return h


def rglru_scan_bwd(x, x_rg_lru, a_rg_lru, a_param, h_saved, grad_out, precision: str = "f64"):
    """(dx, dx_rg_lru, da_rg_lru, dLambda[D]) (restates hawk/scan_fused.py:123-317, :424)."""
    dt = _np_dtype(precision)
    x, xg, ag, lam, hs, go = (
        _prep(v, dt) for v in (x, x_rg_lru, a_rg_lru, a_param, h_saved, grad_out)
    )
    B, T, D = x.shape
    assert hs.shape == x.shape and go.shape == x.shape
    dx, dxg, dag = np.empty_like(x), np.empty_like(x), np.empty_like(x)
    dlam = np.empty(D, dtype=dt)
    fn = getattr(_load(), f"oracle_rglru_scan_bwd_{precision}")
    fn(_ptr(x), _ptr(xg), _ptr(ag), _ptr(lam), _ptr(hs), _ptr(go),
       _ptr(dx), _ptr(dxg), _ptr(dag), _ptr(dlam), B, T, D)
    return dx, dxg, dag, dlam


def conv1d_fwd(x, w, b, state=None, precision: str = "f64"):
    """y[B,T,D] of the causal depthwise temporal conv (restates hawk/external.py:49-95)."""
    dt = _np_dtype(precision)
    x, w, b = _prep(x, dt), _prep(w, dt), _prep(b, dt)
    B, T, D = x.shape
    W = w.shape[0]
    assert w.shape == (W, D) and b.shape == (D,)
    if state is not None:
        state = _prep(state, dt)
        assert state.shape == (B, W - 1, D)
    y = np.empty_like(x)
    fn = getattr(_load(), f"oracle_conv1d_fwd_{precision}")
    fn(_ptr(x), _ptr(w), _ptr(b), _ptr(state), _ptr(y), B, T, D, W)
    return y


def conv1d_bwd(grad_y, x, w, precision: str = "f64"):
    """(dx, dw, db): adjoint of conv1d_fwd with zero history."""
    dt = _np_dtype(precision)
    gy, x, w = _prep(grad_y, dt), _prep(x, dt), _prep(w, dt)
    B, T, D = x.shape
    W = w.shape[0]
    dx = np.empty_like(x)
    dw = np.empty((W, D), dtype=dt)
    db = np.empty(D, dtype=dt)
    fn = getattr(_load(), f"oracle_conv1d_bwd_{precision}")
    fn(_ptr(gy), _ptr(x), _ptr(w), _ptr(dx), _ptr(dw), _ptr(db), B, T, D, W)
    return dx, dw, db


def rglru_step(x, x_rg_lru, a_rg_lru, a_param, state, precision: str = "f64"):
    """One decode step h[B,D] (restates hawk/hawk.py:137-151, :196)."""
    dt = _np_dtype(precision)
    x, xg, ag, lam, st = (_prep(v, dt) for v in (x, x_rg_lru, a_rg_lru, a_param, state))
    B, D = x.shape
    h = np.empty_like(x)
    fn = getattr(_load(), f"oracle_rglru_step_{precision}")
    fn(_ptr(x), _ptr(xg), _ptr(ag), _ptr(lam), _ptr(st), _ptr(h), B, D)
    return h


def conv1d_step(conv_state, x_new, w, b, precision: str = "f64"):
    """One decode step of the conv: returns (y[B,D], new_state[B,W-1,D]).

    Restates hawk/hawk.py:169-179 with hawk/cache.py:37-43.
    """
    dt = _np_dtype(precision)
    st = np.array(conv_state, dtype=dt, order="C", copy=True)
    xn, w, b = _prep(x_new, dt), _prep(w, dt), _prep(b, dt)
    B, D = xn.shape
    W = w.shape[0]
    assert st.shape == (B, W - 1, D)
    y = np.empty_like(xn)
    fn = getattr(_load(), f"oracle_conv1d_step_{precision}")
    fn(_ptr(st), _ptr(xn), _ptr(w), _ptr(b), _ptr(y), B, D, W)
    return y, st


# ---------------------------------------------------------------------------------------
# Scan followed by the block's gate, out = gelu(y) * h (restates Hawk.epilogue before its
# projection, hawk/hawk.py:134-135: F.gelu with its default, the exact erf form).
# ---------------------------------------------------------------------------------------
def gelu(y):
    """y * Phi(y), Phi the standard normal CDF (= 0.5 (1 + erf(y / sqrt 2)))."""
    from scipy.special import ndtr

    y = np.asarray(y, dtype=np.float64)
    return y * ndtr(y)


def gelu_grad(y):
    """d gelu / dy = Phi(y) + y exp(-y^2 / 2) / sqrt(2 pi)."""
    from scipy.special import ndtr

    y = np.asarray(y, dtype=np.float64)
    return ndtr(y) + y * np.exp(-0.5 * y * y) / np.sqrt(2.0 * np.pi)


def rglru_scan_gated_fwd(x, x_rg_lru, a_rg_lru, a_param, y):
    """(h, out) with out = gelu(y) * h; fp64."""
    h = rglru_scan_fwd(x, x_rg_lru, a_rg_lru, a_param)
    return h, gelu(y) * h


def rglru_scan_gated_bwd(x, x_rg_lru, a_rg_lru, a_param, y, h_saved, grad_out):
    """(dx, dx_rg_lru, da_rg_lru, dLambda, dy) for out = gelu(y) * h; fp64.

    The product rule in front of rglru_scan_bwd: the gradient reaching h is
    grad_out * gelu(y), and dy = grad_out * h * gelu'(y) with the saved h.
    """
    go = np.asarray(grad_out, dtype=np.float64)
    hs = np.asarray(h_saved, dtype=np.float64)
    dy = go * hs * gelu_grad(y)
    dx, dxg, dag, dlam = rglru_scan_bwd(x, x_rg_lru, a_rg_lru, a_param, hs, go * gelu(y))
    return dx, dxg, dag, dlam, dy


# ---------------------------------------------------------------------------------------
# Block-diagonal gate projection (restates hawk/external.py:224-233): per block h,
# y[..., h, j] = sum_i x[..., h, i] w[h, i, j] + b[h, j].
# ---------------------------------------------------------------------------------------
def block_diagonal_linear(x, w, b=None):
    """x [..., D], w [nb, bw, bw], b [nb, bw] or [D] or None -> [..., D]; fp64."""
    x = np.asarray(x, dtype=np.float64)
    w = np.asarray(w, dtype=np.float64)
    nb, bw, _ = w.shape
    assert x.shape[-1] == nb * bw and w.shape == (nb, bw, bw)
    y = np.empty_like(x).reshape(-1, nb, bw)
    xb = x.reshape(-1, nb, bw)
    for h in range(nb):
        y[:, h, :] = xb[:, h, :] @ w[h]
    if b is not None:
        y = y + np.asarray(b, dtype=np.float64).reshape(1, nb, bw)
    return y.reshape(x.shape)


def block_diagonal_linear_bwd(x, w, grad_y):
    """(dx, dw, db) of block_diagonal_linear; fp64."""
    x = np.asarray(x, dtype=np.float64)
    w = np.asarray(w, dtype=np.float64)
    gy = np.asarray(grad_y, dtype=np.float64)
    nb, bw, _ = w.shape
    xb, gb = x.reshape(-1, nb, bw), gy.reshape(-1, nb, bw)
    dx = np.empty_like(xb)
    dw = np.empty_like(w)
    for h in range(nb):
        dx[:, h, :] = gb[:, h, :] @ w[h].T
        dw[h] = xb[:, h, :].T @ gb[:, h, :]
    return dx.reshape(x.shape), dw, gb.sum(axis=0)
