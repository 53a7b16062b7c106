"""Decode-time state of one Hawk layer.

Same attribute and method names as upstream's ``RNNCache`` (hawk/cache.py:4-46):
``recc_state`` [B,1,D] and ``conv_state`` [B,W-1,D] in bf16, filled with NaN until first
written, ``current_cache_size``, ``update_cache`` and ``update_conv_cache``.  Two things
are generalised: any batch size B (upstream asserts B == 1) and any temporal conv width
(upstream ignores its ``temporal_conv_width`` argument and always uses 4).  With B == 1
and width 4 the buffers are exactly upstream's.

The decode kernels read and write ``recc_state`` / ``conv_state`` in place and need them
contiguous.  This package never re-binds them, but upstream's own ``Hawk.forward`` does
(``layer_past.conv_state = x[:, -3:, ...]``, hawk/hawk.py:174, a strided view of the input
projection), and its torch-only decode branch works on such a view; ``own_buffers`` turns a
re-bound view back into a contiguous buffer of the cache's own before a kernel touches it.
"""

from __future__ import annotations

import torch


class RNNCache:
    def __init__(
        self,
        state_dim: int,
        device: torch.device,
        temporal_conv_width: int = 4,
        batch_size: int = 1,
        dtype: torch.dtype = torch.bfloat16,
    ):
        assert temporal_conv_width >= 1
        self.temporal_conv_width = temporal_conv_width
        self.conv_cache_size = temporal_conv_width - 1
        self.state_dim = state_dim
        self.batch_size = batch_size
        self.device = device
        self.current_cache_size = 0
        self.recc_state = torch.full((batch_size, 1, state_dim), float("nan"), dtype=dtype, device=device)
        self.conv_state = torch.full(
            (batch_size, self.conv_cache_size, state_dim), float("nan"), dtype=dtype, device=device
        )

    def _check_row(self, new_state: torch.Tensor) -> None:
        assert new_state.ndim == 3, f"expected [B,1,D], got {tuple(new_state.shape)}"
        assert new_state.shape[0] == self.batch_size, (
            f"cache was built for batch {self.batch_size}, got {new_state.shape[0]}"
        )
        assert new_state.shape[1] == 1
        assert new_state.shape[2] == self.state_dim

    def update_cache(self, new_state: torch.Tensor) -> None:
        """Store the recurrent state h_t [B,1,D] (rounded to the cache dtype)."""
        self._check_row(new_state)
        self.recc_state.copy_(new_state)
        self.current_cache_size = 1

    def update_conv_cache(self, new_state: torch.Tensor) -> None:
        """Shift the conv window up by one row and append new_state [B,1,D]."""
        self._check_row(new_state)
        if self.conv_cache_size == 0:
            return
        if self.conv_cache_size > 1:
            self.conv_state[:, :-1, :] = self.conv_state[:, 1:, :].clone()
        self.conv_state[:, -1:, :] = new_state

    def own_buffers(self) -> None:
        """Make ``recc_state`` and ``conv_state`` contiguous tensors that the cache alone
        refers to (a copy is made only for a buffer that was re-bound to a strided view)."""
        if not self.conv_state.is_contiguous():
            self.conv_state = self.conv_state.contiguous()
        if not self.recc_state.is_contiguous():
            self.recc_state = self.recc_state.contiguous()

    def seed_conv_state(self, x: torch.Tensor) -> None:
        """Prefill: keep the last W-1 pre-conv rows of x [B,T,D]; a shorter prompt is
        left-padded with zeros (upstream keeps ``x[:, -3:]``, hawk/hawk.py:174, whose
        missing rows the conv treats as zeros)."""
        assert x.shape[0] == self.batch_size and x.shape[2] == self.state_dim
        keep = min(self.conv_cache_size, x.shape[1])
        self.conv_state.zero_()
        if keep > 0:
            self.conv_state[:, self.conv_cache_size - keep:, :] = x[:, x.shape[1] - keep:, :]

    def __repr__(self) -> str:
        return (
            f"RNNCache: {self.current_cache_size=}, {self.state_dim=}, "
            f"{self.temporal_conv_width=}, {self.batch_size=}"
        )
