"""Hawk language model assembled around the HIP scan / conv / decode kernels.

This is the harness that calls the hot path the way upstream's model does
(hawk/hawk.py:89-303): same constructor arguments, same forward signatures, same
parameter names and shapes (so an upstream ``state_dict`` loads unchanged), same
zero-initialised output projections.  The dense projections and norms are ordinary
PyTorch-ROCm modules (library GEMMs); the loss is plain ``F.cross_entropy``.

What differs from upstream is confined to the recurrent block:

* prefill and training call ``Conv1D`` and the scan from this package; with
  ``HawkConfig.fused_epilogue`` (default) the scan kernel also applies the block's gate,
  ``gelu(y) * h``, and its backward also produces the gate's gradient;
* decode (``use_cache=True`` with a warm ``RNNCache``) issues two fused kernels per layer
  (conv window roll + conv; gate biases + RG-LRU state update + output gate) instead of
  about thirty eager ones, works for any batch size, and evaluates the two gate
  projections once instead of twice.
"""

from __future__ import annotations

import math
from dataclasses import dataclass
from typing import List, Optional, Tuple

import torch
import torch.nn as nn
import torch.nn.functional as F

from .cache import RNNCache
from .external import (
    BlockDiagonalLinear,
    Conv1D,
    decode_core_step,
    decode_core_supported,
    gate_projections,
    gate_projections_supported,
    rglru_step,
    rglru_step_gated,
    rnn_param_init,
    temporal_conv1d,
    temporal_conv1d_step,
)
from .scan_fused import (
    block_core_layout_ok,
    fused_linear_scan,
    fused_linear_scan_gated,
    recurrent_block_core,
    recurrent_core,
)


@dataclass
class HawkConfig:
    vocab_size: int
    hidden_size: int
    intermediate_size: int
    num_hidden_layers: int
    recurrent_size: int
    num_blocks: int
    conv_width: int = 4
    # accepted for compatibility with upstream's README snippet; only False is implemented
    post_norm: bool = False
    # not an upstream field: apply gelu(y) * h inside the scan kernels (hawk/hawk.py:134-135)
    fused_epilogue: bool = True
    # not an upstream field: both gate projections in one matrix-core kernel when the arithmetic
    # is bf16 anyway (bf16 tensors or bf16 autocast); hawk/hawk.py:181-182
    fused_gates: bool = True
    # not an upstream field: with both of the above, a decode step's conv, projections, state
    # update and output gate as one launch (hawk/hawk.py:137-151, :169-182, :196-198)
    fused_decode_core: bool = True
    # not an upstream field: with fused_epilogue and fused_gates, a sequence's conv, projections,
    # scan and output gate as one autograd node that reads both halves of the input projection
    # in place and returns that projection's gradient as one tensor (hawk/hawk.py:163-186)
    fused_block_core: bool = True

    def __post_init__(self):
        if self.post_norm:
            raise NotImplementedError("post_norm=True is not implemented (upstream has no such path either)")


def lecun_init(w: torch.Tensor, d_in: int) -> None:
    nn.init.normal_(w, mean=0.0, std=1.0 / math.sqrt(d_in))


class RMSNorm(nn.Module):
    def __init__(self, dim: int, eps: float = 1e-6):
        super().__init__()
        self.eps = eps
        self.weight = nn.Parameter(torch.ones(dim))

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        # hawk/hawk.py:53-58 normalises in fp32, rounds to x's dtype and multiplies by the weight,
        # about eight eager kernels.  The library's rms_norm does it in one, in fp32 throughout
        # (one rounding less), with the reference's output dtype: x's when the weight has it,
        # fp32 when the weight is an fp32 parameter and x is not.
        if self.weight.dtype == x.dtype:
            return F.rms_norm(x, (x.shape[-1],), self.weight, self.eps)
        return F.rms_norm(x.float(), (x.shape[-1],), self.weight.float(), self.eps)


class MLP(nn.Module):
    """Gated-GeLU feed-forward block."""

    def __init__(self, config: HawkConfig):
        super().__init__()
        self.hidden_size = config.hidden_size
        self.intermediate_size = config.intermediate_size
        self.gate_up_proj = nn.Linear(config.hidden_size, 2 * config.intermediate_size, bias=False)
        self.resid_proj = nn.Linear(config.intermediate_size, config.hidden_size, bias=False)
        self.reset_parameters()

    def reset_parameters(self) -> None:
        lecun_init(self.gate_up_proj.weight, self.hidden_size)
        nn.init.zeros_(self.resid_proj.weight)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        gate, up = self.gate_up_proj(x).chunk(2, dim=-1)
        return self.resid_proj(F.gelu(gate) * up)


class Hawk(nn.Module):
    """Recurrent block: in-projection, temporal conv, gated linear recurrence, gated out-projection."""

    def __init__(self, config: HawkConfig, use_cache: bool = False):
        super().__init__()
        self.config = config
        self.use_cache = use_cache
        R = config.recurrent_size
        self.input_xy = nn.Linear(config.hidden_size, 2 * R, bias=False)
        self.rg_lru_input_gate = BlockDiagonalLinear(width=R, num_blocks=config.num_blocks)
        self.rg_lru_a_gate = BlockDiagonalLinear(width=R, num_blocks=config.num_blocks)
        self.rg_lru_a_param = nn.Parameter(torch.empty([R], dtype=torch.float32))
        self.resid_proj = nn.Linear(R, config.hidden_size, bias=False)
        self.conv1d = Conv1D(width=R, temporal_width=config.conv_width)
        self.reset_parameters()

    def reset_parameters(self) -> None:
        rnn_param_init(self.rg_lru_a_param, min_rad=0.9, max_rad=0.999)
        lecun_init(self.input_xy.weight, self.config.hidden_size)
        nn.init.zeros_(self.resid_proj.weight)

    def forward(self, x: torch.Tensor, layer_past: Optional[RNNCache]) -> Tuple[torch.Tensor, Optional[RNNCache]]:
        warm = self.use_cache and layer_past is not None and layer_past.current_cache_size > 0
        xy = self.input_xy(x)
        branch, gate_branch = xy.chunk(2, dim=-1)

        if warm:
            # One new token per batch row.  (Upstream accepts more and silently keeps only the
            # last position, hawk/hawk.py:178-179, with a conv window that then spans the new
            # rows; nothing sensible can be returned for the other positions, so refuse.)
            assert layer_past is not None
            if x.shape[1] != 1:
                raise ValueError(
                    f"a warm cache takes one new token per call, got {x.shape[1]}; "
                    "feed longer inputs with a fresh RNNCache (prefill)"
                )
            layer_past.own_buffers()
            fused_gates = self.config.fused_gates and gate_projections_supported(branch, self.rg_lru_input_gate)
            gate_branch = gate_branch[:, -1:, :]
            layer_past.current_cache_size = 1
            if (fused_gates and self.config.fused_epilogue and self.config.fused_decode_core
                    and decode_core_supported(branch, self.conv1d, self.rg_lru_input_gate, layer_past.conv_state)):
                gated = decode_core_step(layer_past.conv_state, branch[:, -1:, :], self.conv1d,
                                         self.rg_lru_input_gate, self.rg_lru_a_gate, self.rg_lru_a_param,
                                         layer_past.recc_state, gate_branch)
                return self.resid_proj(gated), layer_past
            if fused_gates:
                u = temporal_conv1d_step(layer_past.conv_state, branch[:, -1:, :], self.conv1d.w, self.conv1d.b,
                                         torch.bfloat16)
                xg, ag = gate_projections(u, self.rg_lru_input_gate, self.rg_lru_a_gate, torch.bfloat16)
                bias_i = bias_a = None  # already added by the projection kernel
            else:
                u = self.conv1d.step(layer_past.conv_state, branch[:, -1:, :])
                xg = self.rg_lru_input_gate(u, add_bias=False)
                ag = self.rg_lru_a_gate(u, add_bias=False)
                bias_i, bias_a = self.rg_lru_input_gate.b, self.rg_lru_a_gate.b
            if self.config.fused_epilogue:
                gated = rglru_step_gated(u, xg, ag, self.rg_lru_a_param, layer_past.recc_state, gate_branch,
                                         bias_i=bias_i, bias_a=bias_a)
                return self.resid_proj(gated), layer_past
            if bias_i is not None:
                xg, ag = xg + bias_i.reshape(-1), ag + bias_a.reshape(-1)
            h = rglru_step(u, xg, ag, self.rg_lru_a_param, layer_past.recc_state)
            cache = layer_past
        else:
            if self.use_cache:
                assert layer_past is not None, "use_cache=True needs one RNNCache per layer in layer_past"
                layer_past.seed_conv_state(branch)
            cache = layer_past if self.use_cache else None
            if self.config.fused_gates and gate_projections_supported(branch, self.rg_lru_input_gate):
                if (self.config.fused_epilogue and self.config.fused_block_core and block_core_layout_ok(xy)):
                    # conv, projections, scan and output gate as one autograd node on xy itself
                    gated, h_last = recurrent_block_core(xy, self.conv1d, self.rg_lru_input_gate,
                                                         self.rg_lru_a_gate, self.rg_lru_a_param,
                                                         return_last_state=True)
                    if self.use_cache:
                        layer_past.update_cache(h_last)
                    return self.resid_proj(gated), cache
                # bf16 end to end: upstream's gate einsums (under autocast) and its scan
                # (cast_inputs, hawk/scan_fused.py:428) round the conv output to bf16 anyway
                u = temporal_conv1d(branch, self.conv1d.w, self.conv1d.b, torch.bfloat16)
                if self.config.fused_epilogue:
                    # projections, scan and output gate as one autograd node
                    gated, h_last = recurrent_core(u, self.rg_lru_input_gate, self.rg_lru_a_gate,
                                                   self.rg_lru_a_param, gate_branch, return_last_state=True)
                    if self.use_cache:
                        layer_past.update_cache(h_last)
                    return self.resid_proj(gated), cache
                xg, ag = gate_projections(u, self.rg_lru_input_gate, self.rg_lru_a_gate, torch.bfloat16)
            else:
                u = self.conv1d(branch)
                xg, ag = self.rg_lru_input_gate(u), self.rg_lru_a_gate(u)
            gates = (xg, ag, self.rg_lru_a_param.float())
            if self.config.fused_epilogue:
                gated, h_last = fused_linear_scan_gated(u, *gates, gate_branch, return_last_state=True)
                if self.use_cache:
                    layer_past.update_cache(h_last)
                return self.resid_proj(gated), cache
            h = fused_linear_scan(u, *gates)
            if self.use_cache:
                layer_past.update_cache(h[:, -1:, :])

        return self.resid_proj(F.gelu(gate_branch) * h), cache


class RNNLayer(nn.Module):
    """Pre-norm residual layer: recurrent block, then MLP."""

    def __init__(self, config: HawkConfig, use_cache: bool = False):
        super().__init__()
        self.use_cache = use_cache
        self.recc = Hawk(config, use_cache)
        self.mlp = MLP(config)
        self.input_norm = RMSNorm(config.hidden_size)
        self.post_recurrent_norm = RMSNorm(config.hidden_size)

    def forward(self, hidden_states: torch.Tensor, layer_past: Optional[RNNCache] = None):
        mixed, cache = self.recc(x=self.input_norm(hidden_states), layer_past=layer_past)
        hidden_states = hidden_states + mixed
        hidden_states = hidden_states + self.mlp(self.post_recurrent_norm(hidden_states))
        return hidden_states, cache


class HawkModel(nn.Module):
    """Embedding, ``num_hidden_layers`` RNNLayers, final norm, LM head.

    ``forward(input_ids, labels=None, layer_past=None)`` returns, as upstream
    (hawk/hawk.py:260-303): ``(logits, caches)`` when ``use_cache``; the next-token loss
    when ``labels`` is given; logits otherwise.
    """

    def __init__(self, config: HawkConfig, use_cache: bool = False):
        super().__init__()
        self.config = config
        self.use_cache = use_cache
        self.embed_tokens = nn.Embedding(config.vocab_size, config.hidden_size)
        self.layers = nn.ModuleList([RNNLayer(config, use_cache) for _ in range(config.num_hidden_layers)])
        self.norm = RMSNorm(config.hidden_size)
        self.lm_head = nn.Linear(config.hidden_size, config.vocab_size, bias=False)
        self.reset_parameters()

    def reset_parameters(self) -> None:
        lecun_init(self.embed_tokens.weight, self.config.hidden_size)
        nn.init.zeros_(self.lm_head.weight)

    def new_cache(self, batch_size: int = 1, device=None) -> List[RNNCache]:
        """One empty RNNCache per layer, for ``use_cache=True`` prefill and decode."""
        device = device if device is not None else self.embed_tokens.weight.device
        return [
            RNNCache(self.config.recurrent_size, device, self.config.conv_width, batch_size=batch_size)
            for _ in self.layers
        ]

    def forward(
        self,
        input_ids: Optional[torch.LongTensor] = None,
        labels: Optional[torch.LongTensor] = None,
        layer_past: Optional[List[Optional[RNNCache]]] = None,
    ):
        if layer_past is None:
            layer_past = [None] * len(self.layers)
        assert isinstance(layer_past, list) and len(layer_past) == len(self.layers)

        hidden_states = self.embed_tokens(input_ids)
        caches = []
        for layer, past in zip(self.layers, layer_past):
            hidden_states, cache = layer(hidden_states, layer_past=past)
            caches.append(cache)
        hidden_states = self.norm(hidden_states)

        if self.use_cache:
            return self.lm_head(hidden_states), caches
        if labels is not None:
            logits = self.lm_head(hidden_states[..., :-1, :])
            return F.cross_entropy(logits.reshape(-1, logits.size(-1)).float(), labels[..., 1:].reshape(-1))
        return self.lm_head(hidden_states)
