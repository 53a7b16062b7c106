"""Writes ``rglru_independent.npz``: RG-LRU forward values and gradients from an implementation
that shares no code with this repository or with its oracle.

The generator is the pure-PyTorch ``RecurrentGemmaRglru`` module of the installed
``transformers`` package (same DeepMind lineage as hawk/scan_fused.py: identical gate
parameterisation, identical clipped square-root derivative, a plain Python loop over time).
It is used unmodified.  Two things need care:

* that module resets the state and sets the input multiplier to 1 wherever
  ``position_ids == 0``; Hawk has no such reset (hawk/scan_fused.py:77-81), so positions
  start at 1;
* it derives both gate logits from the activations through block-diagonal weights.  To
  drive the two logits independently of ``x``, every head is given 3n channels: the first n
  carry ``x``, the next n carry the wanted ``x_rg_lru`` and the last n the wanted
  ``a_rg_lru``; the gate weights are 0/1 selection matrices routing channel ``n + j`` (or
  ``2n + j``) to the gate of channel ``j``.  Gradients of the activations on the three
  channel groups are then exactly ``dx``, ``dx_rg_lru`` and ``da_rg_lru``.

Run from the repository root (CPU only, a few seconds):

    python tests/golden/make_rglru_fixture.py

The fixture holds data only: inputs, ``h``, the upstream gradient, and the four gradients.
"""

from __future__ import annotations

import os
from types import SimpleNamespace

import numpy as np
import torch
from transformers.models.recurrent_gemma.modeling_recurrent_gemma import RecurrentGemmaRglru

HERE = os.path.dirname(os.path.abspath(__file__))


def main() -> None:
    torch.manual_seed(20240607)
    B, T, heads, n = 2, 37, 2, 6
    bw = 3 * n
    D = heads * n
    cfg = SimpleNamespace(num_attention_heads=heads, lru_width=heads * bw)
    mod = RecurrentGemmaRglru(cfg).double()

    x = torch.randn(B, T, D, dtype=torch.float64)
    xg = 1.5 * torch.randn(B, T, D, dtype=torch.float64)
    ag = 1.5 * torch.randn(B, T, D, dtype=torch.float64)
    # a^8 = sigmoid(-Lambda)^8 spread over (0.5, 0.9999); the last two channels are pushed to
    # softplus(Lambda) ~ 2e-9 so that 1 - a^2 < 2.5e-7 and the clipped derivative is what acts
    u = torch.linspace(0.5, 0.9999, D, dtype=torch.float64)
    lam = torch.log(u ** (-1.0 / 8.0) - 1.0)
    lam[-2:] = -20.0

    act = torch.zeros(B, T, heads, bw, dtype=torch.float64)
    act[..., :n] = x.reshape(B, T, heads, n)
    act[..., n : 2 * n] = xg.reshape(B, T, heads, n)
    act[..., 2 * n :] = ag.reshape(B, T, heads, n)
    act = act.reshape(B, T, heads * bw).requires_grad_(True)

    with torch.no_grad():
        wi = torch.zeros(heads, bw, bw, dtype=torch.float64)
        wa = torch.zeros(heads, bw, bw, dtype=torch.float64)
        for j in range(n):
            wi[:, n + j, j] = 1.0
            wa[:, 2 * n + j, j] = 1.0
        mod.input_gate_weight.copy_(wi)
        mod.recurrent_gate_weight.copy_(wa)
        mod.input_gate_bias.zero_()
        mod.recurrent_gate_bias.zero_()
        lam_wide = torch.zeros(heads, bw, dtype=torch.float64)
        lam_wide[:, :n] = lam.reshape(heads, n)
        mod.recurrent_param.copy_(lam_wide.reshape(-1))

    pos = torch.arange(1, T + 1)[None, :].expand(B, T)
    h_wide = mod(act, pos)
    h = h_wide.reshape(B, T, heads, bw)[..., :n].reshape(B, T, D)

    gout = torch.randn(B, T, D, dtype=torch.float64)
    (h * gout).sum().backward()
    g = act.grad.reshape(B, T, heads, bw)
    dx = g[..., :n].reshape(B, T, D)
    dxg = g[..., n : 2 * n].reshape(B, T, D)
    dag = g[..., 2 * n :].reshape(B, T, D)
    dlam = mod.recurrent_param.grad.reshape(heads, bw)[:, :n].reshape(D)

    np.savez(
        os.path.join(HERE, "rglru_independent.npz"),
        x=x.numpy(), x_rg_lru=xg.numpy(), a_rg_lru=ag.numpy(), a_param=lam.numpy(),
        h=h.detach().numpy(), grad_out=gout.numpy(),
        dx=dx.numpy(), dx_rg_lru=dxg.numpy(), da_rg_lru=dag.numpy(), da_param=dlam.numpy(),
    )
    print("wrote rglru_independent.npz", "B,T,D =", (B, T, D))


if __name__ == "__main__":
    main()
