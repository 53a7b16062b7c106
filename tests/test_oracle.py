"""Pins the CPU oracle (oracle/) by facts that do not come from the oracle itself.

Upstream holds no tests, fixtures or golden vectors, so each function of the oracle is
pinned by mathematics: closed forms, a library routine, an independent derivation by
automatic differentiation, finite differences, and special cases, chosen so that a dropped
term, a wrong sign or an off-by-one time index fails at least one of them.  A fixture written
by an unrelated third-party implementation is checked in test_golden.py.
"""

import numpy as np
import pytest
import scipy.signal
import torch

import oracle
from oracle import rglru_torch
from conftest import make_scan_inputs, max_rel


def _sigmoid(v):
    return 1.0 / (1.0 + np.exp(-v))


def _softplus(v):
    return np.log1p(np.exp(v))


# ------------------------------------------------------------------------------ scan forward
def test_scan_fwd_constant_gates_is_a_first_order_iir_filter():
    """With time-constant gate logits, alpha and m are constants per channel and
    h = lfilter([1], [1, -alpha], m*i*x): a textbook one-pole filter."""
    rng = np.random.default_rng(1)
    B, T, D = 2, 300, 5
    x = rng.standard_normal((B, T, D))
    xg = np.broadcast_to(rng.standard_normal((1, 1, D)), (B, T, D)).copy()
    ag = np.broadcast_to(rng.standard_normal((1, 1, D)), (B, T, D)).copy()
    lam = rng.uniform(-6.0, 1.0, size=D)
    h = oracle.rglru_scan_fwd(x, xg, ag, lam)
    for d in range(D):
        alpha = np.exp(-8.0 * _sigmoid(ag[0, 0, d]) * _softplus(lam[d]))
        beta = np.sqrt(1.0 - alpha**2) * _sigmoid(xg[0, 0, d]) * x[:, :, d]
        ref = scipy.signal.lfilter([1.0], [1.0, -alpha], beta, axis=1)
        np.testing.assert_allclose(h[:, :, d], ref, rtol=1e-11, atol=1e-13)


def test_scan_fwd_gate_extremes():
    x, xg, ag, lam, _ = make_scan_inputs(1, 40, 6, seed=2)
    # r -> 0: alpha = 1, m = 0, so beta = 0 and h stays at its initial value 0
    h = oracle.rglru_scan_fwd(x, xg, np.full_like(ag, -800.0), lam)
    assert np.all(h == 0.0)
    # alpha -> 0 (r = 1, very large softplus): no memory, h_t = i_t x_t
    h = oracle.rglru_scan_fwd(x, xg, np.full_like(ag, 50.0), np.full_like(lam, 30.0))
    np.testing.assert_allclose(h, _sigmoid(xg) * x, rtol=1e-12)


def test_scan_fwd_first_step_has_no_reset_and_matches_torch_loop():
    """h_0 = m_0 i_0 x_0 (no 'multiplier = 1 at position 0'); and the C loops agree with
    the independent torch loop over the one-token decode arithmetic."""
    x, xg, ag, lam, _ = make_scan_inputs(3, 50, 16, seed=3)
    h = oracle.rglru_scan_fwd(x, xg, ag, lam)
    alpha0 = np.exp(-8.0 * _sigmoid(ag[:, 0]) * _softplus(lam))
    np.testing.assert_allclose(h[:, 0], np.sqrt(1 - alpha0**2) * _sigmoid(xg[:, 0]) * x[:, 0], rtol=1e-12)
    t = [torch.from_numpy(v) for v in (x, xg, ag, lam)]
    ref = rglru_torch.rglru_scan_loop(*t).numpy()
    np.testing.assert_allclose(h, ref, rtol=1e-12, atol=1e-14)


def test_scan_fwd_is_linear_in_x():
    x, xg, ag, lam, _ = make_scan_inputs(1, 64, 8, seed=4)
    x2 = np.random.default_rng(5).standard_normal(x.shape)
    lhs = oracle.rglru_scan_fwd(2.0 * x - 3.0 * x2, xg, ag, lam)
    rhs = 2.0 * oracle.rglru_scan_fwd(x, xg, ag, lam) - 3.0 * oracle.rglru_scan_fwd(x2, xg, ag, lam)
    np.testing.assert_allclose(lhs, rhs, rtol=1e-11, atol=1e-12)


# ----------------------------------------------------------------------------- scan backward
@pytest.mark.parametrize("shape,seed", [((2, 37, 8), 0), ((1, 1, 4), 1), ((1, 2, 4), 2), ((3, 130, 3), 3)])
def test_scan_bwd_matches_autograd_of_the_torch_loop(shape, seed):
    """Analytic reverse-time formulas (C) against automatic differentiation (torch) of an
    independently written forward: two derivations, one answer.  Includes T = 1 and 2."""
    B, T, D = shape
    x, xg, ag, lam, gout = make_scan_inputs(B, T, D, seed=seed)
    t = [torch.from_numpy(v) for v in (x, xg, ag, lam, gout)]
    h_ref, *g_ref = rglru_torch.rglru_scan_fwd_bwd(*t)
    h = oracle.rglru_scan_fwd(x, xg, ag, lam)
    got = oracle.rglru_scan_bwd(x, xg, ag, lam, h, gout)
    for name, a, b in zip(("dx", "dx_rg_lru", "da_rg_lru", "da_param"), got, g_ref):
        assert max_rel(a, b.numpy()) < 1e-12, name


def test_scan_bwd_matches_finite_differences():
    """Central differences of L = sum(gout * h) away from the sqrt-derivative clip."""
    B, T, D = 1, 9, 3
    x, xg, ag, lam, gout = make_scan_inputs(B, T, D, seed=7, lo=0.3, hi=0.9)
    h = oracle.rglru_scan_fwd(x, xg, ag, lam)
    dx, dxg, dag, dlam = oracle.rglru_scan_bwd(x, xg, ag, lam, h, gout)

    def loss(x_, xg_, ag_, lam_):
        return float((gout * oracle.rglru_scan_fwd(x_, xg_, ag_, lam_)).sum())

    eps = 1e-6
    args = [x, xg, ag, lam]
    for which, grad in enumerate((dx, dxg, dag, dlam)):
        flat = args[which].reshape(-1)
        for idx in range(0, flat.size, max(1, flat.size // 7)):
            plus = [a.copy() for a in args]
            minus = [a.copy() for a in args]
            plus[which].reshape(-1)[idx] += eps
            minus[which].reshape(-1)[idx] -= eps
            fd = (loss(*plus) - loss(*minus)) / (2 * eps)
            assert abs(fd - grad.reshape(-1)[idx]) < 1e-6 * max(1.0, abs(fd)), (which, idx)


def test_scan_bwd_clip_branch_closed_form():
    """Inside the clip (1 - alpha^2 < 2.5e-7) the sqrt derivative is exactly 1000, so for
    T = 1:  da_rg_lru = r(1-r) (-8 s) * gout * i * x * 1000 * (-2 alpha^2)."""
    D = 4
    lam = np.full(D, -20.0)  # softplus ~ 2.06e-9  =>  1 - alpha^2 ~ 3e-8 r
    x, xg, ag, _, gout = make_scan_inputs(1, 1, D, seed=8)
    s = _softplus(lam)
    r, i = _sigmoid(ag[0, 0]), _sigmoid(xg[0, 0])
    a2 = np.exp(-16.0 * r * s)
    assert np.all(1.0 - a2 < 2.5e-7)
    h = oracle.rglru_scan_fwd(x, xg, ag, lam)
    _, _, dag, dlam = oracle.rglru_scan_bwd(x, xg, ag, lam, h, gout)
    dlog_a = gout[0, 0] * i * x[0, 0] * 1000.0 * (-2.0 * a2)
    np.testing.assert_allclose(dag[0, 0], r * (1 - r) * (-8.0 * s) * dlog_a, rtol=1e-12)
    np.testing.assert_allclose(dlam, dlog_a * (-8.0) * r * _sigmoid(lam), rtol=1e-12)
    # and the autograd path, whose sqrt carries the same bound, agrees there too
    t = [torch.from_numpy(v) for v in (x, xg, ag, lam, gout)]
    _, _, _, dag_t, dlam_t = rglru_torch.rglru_scan_fwd_bwd(*t)
    np.testing.assert_allclose(dag, dag_t.numpy(), rtol=1e-10)
    np.testing.assert_allclose(dlam, dlam_t.numpy(), rtol=1e-10)


def test_scan_bwd_uses_previous_state_not_current():
    """d_alpha_t multiplies h_{t-1}: shifting h_saved by one row must change da_rg_lru."""
    x, xg, ag, lam, gout = make_scan_inputs(1, 6, 2, seed=9)
    h = oracle.rglru_scan_fwd(x, xg, ag, lam)
    good = oracle.rglru_scan_bwd(x, xg, ag, lam, h, gout)[2]
    shifted = oracle.rglru_scan_bwd(x, xg, ag, lam, np.roll(h, -1, axis=1), gout)[2]
    assert max_rel(shifted, good) > 1e-3
    # row 0 has no d_alpha term at all, so it does not depend on h_saved
    np.testing.assert_allclose(shifted[:, 0], good[:, 0], rtol=1e-13)


# --------------------------------------------------------------------------------------- conv
@pytest.mark.parametrize("W", [1, 2, 4, 7])
@pytest.mark.parametrize("T", [1, 3, 25])
def test_conv_fwd_bwd_match_library_conv1d(W, T):
    rng = np.random.default_rng(10 + W + T)
    B, D = 2, 6
    x = rng.standard_normal((B, T, D))
    w = rng.standard_normal((W, D)) * 0.5
    b = rng.standard_normal(D)
    gy = rng.standard_normal((B, T, D))
    xt, wt, bt = (torch.from_numpy(v).requires_grad_(True) for v in (x, w, b))
    y_ref = rglru_torch.conv1d_library(xt, wt, bt)
    y_ref.backward(torch.from_numpy(gy))
    np.testing.assert_allclose(oracle.conv1d_fwd(x, w, b), y_ref.detach().numpy(), rtol=1e-12, atol=1e-13)
    dx, dw, db = oracle.conv1d_bwd(gy, x, w)
    np.testing.assert_allclose(dx, xt.grad.numpy(), rtol=1e-12, atol=1e-13)
    np.testing.assert_allclose(dw, wt.grad.numpy(), rtol=1e-12, atol=1e-13)
    np.testing.assert_allclose(db, bt.grad.numpy(), rtol=1e-12, atol=1e-13)


def test_conv_weight_row_order():
    """w[W-1] multiplies the current row, w[0] the oldest (hawk/external.py:88 upstream)."""
    D, W, T = 3, 4, 6
    x = np.zeros((1, T, D))
    x[0, 2] = 1.0  # impulse at t = 2
    w = np.arange(W * D, dtype=np.float64).reshape(W, D) + 1.0
    y = oracle.conv1d_fwd(x, w, np.zeros(D))
    for s in range(W):
        if 2 + s < T:
            np.testing.assert_array_equal(y[0, 2 + s], w[W - 1 - s])
    assert np.all(y[0, :2] == 0.0)


def test_conv_with_state_equals_conv_of_the_joined_sequence():
    rng = np.random.default_rng(11)
    B, T, D, W = 2, 9, 5, 4
    full = rng.standard_normal((B, T + W - 1, D))
    w, b = rng.standard_normal((W, D)), rng.standard_normal(D)
    y_full = oracle.conv1d_fwd(full, w, b)
    y_state = oracle.conv1d_fwd(full[:, W - 1:], w, b, state=full[:, : W - 1])
    np.testing.assert_allclose(y_state, y_full[:, W - 1:], rtol=1e-13)


# ------------------------------------------------------------------------------ decode steps
def test_prefill_then_step_equals_scan_over_one_more_row():
    x, xg, ag, lam, _ = make_scan_inputs(3, 21, 8, seed=12)
    h_full = oracle.rglru_scan_fwd(x, xg, ag, lam)
    h_prefill = oracle.rglru_scan_fwd(x[:, :-1], xg[:, :-1], ag[:, :-1], lam)
    h_step = oracle.rglru_step(x[:, -1], xg[:, -1], ag[:, -1], lam, h_prefill[:, -1])
    np.testing.assert_allclose(h_step, h_full[:, -1], rtol=1e-12)


def test_conv_step_rolls_state_and_matches_full_conv():
    rng = np.random.default_rng(13)
    B, T, D, W = 2, 12, 4, 4
    x = rng.standard_normal((B, T, D))
    w, b = rng.standard_normal((W, D)), rng.standard_normal(D)
    y_full = oracle.conv1d_fwd(x, w, b)
    state = np.zeros((B, W - 1, D))
    for t in range(T):
        y, new_state = oracle.conv1d_step(state, x[:, t], w, b)
        np.testing.assert_allclose(y, y_full[:, t], rtol=1e-12, atol=1e-13)
        # roll by -1 along time, newest row last (hawk/cache.py:42-43 upstream)
        np.testing.assert_array_equal(new_state[:, :-1], state[:, 1:])
        np.testing.assert_array_equal(new_state[:, -1], x[:, t])
        state = new_state


# ------------------------------------------------------------------------------- fp32 port
def test_f32_port_tracks_f64():
    x, xg, ag, lam, gout = make_scan_inputs(1, 256, 32, seed=14)
    h64 = oracle.rglru_scan_fwd(x, xg, ag, lam)
    h32 = oracle.rglru_scan_fwd(x, xg, ag, lam, precision="f32")
    assert max_rel(h32, h64) < 1e-4
    g64 = oracle.rglru_scan_bwd(x, xg, ag, lam, h64, gout)
    g32 = oracle.rglru_scan_bwd(x, xg, ag, lam, h64, gout, precision="f32")
    for a, b in zip(g32, g64):
        assert max_rel(a, b) < 1e-3


# ------------------------------------------------------------------------------ gated epilogue
def test_gelu_and_its_derivative_match_the_library_routine():
    y = np.concatenate([np.linspace(-9.0, 9.0, 2001), [0.0, -0.0, 1e-8, -1e-8, 30.0, -30.0]])
    t = torch.from_numpy(y).requires_grad_(True)
    g = torch.nn.functional.gelu(t)  # exact (erf) form, the default used at hawk/hawk.py:135
    (dg,) = torch.autograd.grad(g.sum(), t)
    # the library evaluates 0.5 y (1 + erf(y / sqrt 2)), which cancels in the far negative tail;
    # the oracle uses the normal CDF directly, hence the absolute floor
    np.testing.assert_allclose(oracle.gelu(y), g.detach().numpy(), rtol=1e-12, atol=2e-15)
    np.testing.assert_allclose(oracle.gelu_grad(y), dg.numpy(), rtol=1e-10, atol=2e-15)
    # closed-form anchors: gelu(0) = 0, gelu'(0) = 1/2, gelu(y) - gelu(-y) = y
    assert oracle.gelu(0.0) == 0.0 and oracle.gelu_grad(0.0) == 0.5
    np.testing.assert_allclose(oracle.gelu(y) - oracle.gelu(-y), y, rtol=1e-12, atol=1e-12)


def test_gated_scan_matches_autograd_of_the_torch_composition():
    x, xg, ag, lam, gout = make_scan_inputs(2, 19, 6, seed=4)
    y = 1.5 * np.random.default_rng(8).standard_normal(x.shape)
    t = [torch.from_numpy(v).requires_grad_(True) for v in (x, xg, ag, lam, y)]
    h = rglru_torch.rglru_scan_loop(*t[:4])
    out = torch.nn.functional.gelu(t[4]) * h
    grads = torch.autograd.grad(out, t, torch.from_numpy(gout))
    h_o, out_o = oracle.rglru_scan_gated_fwd(x, xg, ag, lam, y)
    assert max_rel(out_o, out.detach().numpy()) < 1e-12
    got = oracle.rglru_scan_gated_bwd(x, xg, ag, lam, y, h_o, gout)
    order = (0, 1, 2, 3, 4)  # dx, dx_rg_lru, da_rg_lru, dLambda, dy
    for k, a in zip(order, got):
        assert max_rel(a, grads[k].numpy()) < 1e-10, k


# ------------------------------------------------------------------------------ gate projections
def test_block_diagonal_linear_equals_a_dense_layer_with_a_block_diagonal_matrix():
    rng = np.random.default_rng(0)
    nb, bw, M = 3, 5, 7
    x = rng.standard_normal((2, M, nb * bw))
    w = rng.standard_normal((nb, bw, bw))
    b = rng.standard_normal((nb, bw))
    dense = np.zeros((nb * bw, nb * bw))
    for h in range(nb):
        dense[h * bw:(h + 1) * bw, h * bw:(h + 1) * bw] = w[h]
    want = x @ dense + b.reshape(-1)
    np.testing.assert_allclose(oracle.block_diagonal_linear(x, w, b), want, rtol=1e-13, atol=1e-13)
    # and the einsum upstream writes (hawk/external.py:230)
    t = torch.einsum("...hi,hij->...hj", torch.from_numpy(x).reshape(2, M, nb, bw), torch.from_numpy(w))
    np.testing.assert_allclose(oracle.block_diagonal_linear(x, w), t.reshape(2, M, -1).numpy(), rtol=1e-13, atol=1e-13)
    # backward against autograd
    xt = torch.from_numpy(x).requires_grad_(True)
    wt = torch.from_numpy(w).requires_grad_(True)
    bt = torch.from_numpy(b).requires_grad_(True)
    y = (torch.einsum("...hi,hij->...hj", xt.reshape(2, M, nb, bw), wt) + bt).reshape(2, M, -1)
    gy = rng.standard_normal(y.shape)
    y.backward(torch.from_numpy(gy))
    dx, dw, db = oracle.block_diagonal_linear_bwd(x, w, gy)
    np.testing.assert_allclose(dx, xt.grad.numpy(), rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(dw, wt.grad.numpy(), rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(db, bt.grad.numpy(), rtol=1e-12, atol=1e-12)
