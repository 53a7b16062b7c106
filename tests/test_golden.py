"""The committed fixture ``tests/golden/rglru_independent.npz`` against the oracle (CPU) and
against the HIP kernels through the C ABI (GPU).

The fixture was written by ``tests/golden/make_rglru_fixture.py`` from an RG-LRU
implementation that shares no code with this repository (a third-party pure-PyTorch module
with a Python loop over time and autograd).  It accumulates the state in fp32, so agreement
is to about 1e-6 of each tensor's scale, not to fp64 round-off.  Its last two channels have
1 - a^2 below 2.5e-7, so the clipped square-root derivative of hawk/scan_fused.py:10-15 is
part of what is compared.
"""

import os

import numpy as np
import pytest
import torch

import oracle
from oracle import rglru_torch
from conftest import max_rel

FIXTURE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "rglru_independent.npz")
GRADS = ("dx", "dx_rg_lru", "da_rg_lru", "da_param")


@pytest.fixture(scope="module")
def golden():
    with np.load(FIXTURE, allow_pickle=False) as f:
        return {k: f[k] for k in f.files}


def test_fixture_exercises_the_clip_branch(golden):
    lam, ag = golden["a_param"], golden["a_rg_lru"]
    softplus = np.log1p(np.exp(lam))
    log_a = -8.0 / (1.0 + np.exp(-ag)) * softplus
    z = -np.expm1(2.0 * log_a)
    assert (4.0 * z[..., -2:] < 1e-6).all() and (4.0 * z[..., :-2] > 1e-6).all()
    assert np.abs(golden["da_param"][-2:]).min() > 0.0


def test_oracle_reproduces_the_independent_fixture(golden):
    g = golden
    h = oracle.rglru_scan_fwd(g["x"], g["x_rg_lru"], g["a_rg_lru"], g["a_param"])
    assert max_rel(h, g["h"]) < 2e-6
    got = oracle.rglru_scan_bwd(g["x"], g["x_rg_lru"], g["a_rg_lru"], g["a_param"], g["h"], g["grad_out"])
    for name, a in zip(GRADS, got):
        assert max_rel(a, g[name]) < 2e-6, (name, max_rel(a, g[name]))
    # the two clipped channels on their own scale, which is 1e-4 of the largest dLambda
    assert max_rel(got[3][-2:], g["da_param"][-2:]) < 1e-4


def test_f32_port_reproduces_the_fixture_away_from_the_cancellation(golden):
    """The scalar fp32 port evaluates 1 - exp(2 log a) as written upstream, which is exactly 0
    in fp32 once |2 log a| < 6e-8; the last two channels sit there, so they are left out."""
    g = {k: (v[..., :-2] if v.ndim else v) for k, v in golden.items()}
    h = oracle.rglru_scan_fwd(g["x"], g["x_rg_lru"], g["a_rg_lru"], g["a_param"], precision="f32")
    assert max_rel(h, g["h"]) < 2e-5
    got = oracle.rglru_scan_bwd(g["x"], g["x_rg_lru"], g["a_rg_lru"], g["a_param"], g["h"], g["grad_out"],
                                precision="f32")
    for name, a in zip(GRADS, got):
        assert max_rel(a, g[name]) < 2e-5, (name, max_rel(a, g[name]))


def test_torch_loop_reproduces_the_independent_fixture(golden):
    g = golden
    t = {k: torch.from_numpy(v) for k, v in g.items()}
    h, *grads = rglru_torch.rglru_scan_fwd_bwd(t["x"], t["x_rg_lru"], t["a_rg_lru"], t["a_param"], t["grad_out"])
    assert max_rel(h.numpy(), g["h"]) < 2e-6
    for name, a in zip(GRADS, grads):
        assert max_rel(a.numpy(), g[name]) < 2e-6, name


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_hip_scan_reproduces_the_independent_fixture(golden, dtype):
    import capi
    from conftest import TOL

    g = golden
    dev = {k: capi.to_dev(g[k], dtype) for k in ("x", "x_rg_lru", "a_rg_lru", "grad_out")}
    lam = capi.to_dev(g["a_param"], "f32")
    h = capi.scan_fwd(dev["x"], dev["x_rg_lru"], dev["a_rg_lru"], lam)
    grads = capi.scan_bwd(dev["x"], dev["x_rg_lru"], dev["a_rg_lru"], lam, h, dev["grad_out"])
    torch.cuda.synchronize()
    tol = TOL[dtype]
    assert max_rel(capi.to_np(h), g["h"]) < tol
    for name, a in zip(GRADS, grads):
        assert max_rel(capi.to_np(a), g[name]) < tol, (name, dtype, max_rel(capi.to_np(a), g[name]))
