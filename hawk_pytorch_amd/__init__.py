"""MI355X-native RG-LRU scan, temporal conv1d and decode kernels for Hawk, with the
operator / module surface of fattorib/hawk-pytorch (``from hawk import HawkModel, HawkConfig``
becomes ``from hawk_pytorch_amd import HawkModel, HawkConfig``)."""

from ._lib import HawkHipError, check_scan_status, release_workspaces
from .cache import RNNCache
from .external import (
    BlockDiagonalLinear,
    Conv1D,
    decode_core_step,
    gate_projections,
    rglru_step,
    rglru_step_gated,
    rnn_param_init,
    temporal_conv1d,
    temporal_conv1d_step,
)
from .hawk import Hawk, HawkConfig, HawkModel, MLP, RMSNorm, RNNLayer
from .scan_fused import (
    DiagonalRecurrence,
    GatedDiagonalRecurrence,
    fused_linear_scan,
    fused_linear_scan_gated,
    recurrent_block_core,
    recurrent_core,
    sequential_scan_backward,
    sequential_scan_forward,
)

__all__ = [
    "BlockDiagonalLinear",
    "Conv1D",
    "DiagonalRecurrence",
    "GatedDiagonalRecurrence",
    "Hawk",
    "HawkConfig",
    "HawkHipError",
    "HawkModel",
    "MLP",
    "RMSNorm",
    "RNNCache",
    "RNNLayer",
    "check_scan_status",
    "decode_core_step",
    "fused_linear_scan",
    "gate_projections",
    "recurrent_block_core",
    "recurrent_core",
    "release_workspaces",
    "fused_linear_scan_gated",
    "rglru_step",
    "rglru_step_gated",
    "rnn_param_init",
    "sequential_scan_backward",
    "sequential_scan_forward",
    "temporal_conv1d",
    "temporal_conv1d_step",
]
