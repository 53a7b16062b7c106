"""ctypes binding of libhawk_hip.so (declared in include/hawk_hip.h).

The library is the product: there is no CPU or eager fallback.  If the shared object
cannot be found or built, or a call reports a non-zero status, an exception is raised.
"""

from __future__ import annotations

import ctypes
import itertools
import math
import os
import threading

import torch

_CSRC = os.path.join(os.path.dirname(os.path.abspath(__file__)), "csrc")
# HAWK_HIP_LIB selects another build of the library (e.g. one compiled with other tile shapes)
LIB_PATH = os.environ.get("HAWK_HIP_LIB") or os.path.join(_CSRC, "libhawk_hip.so")

HAWK_OK = 0
HAWK_ERR_NULL_POINTER = 1
HAWK_ERR_BAD_SHAPE = 2
HAWK_ERR_BAD_DTYPE = 3
HAWK_ERR_WORKSPACE = 4
HAWK_ERR_LAUNCH = 5
HAWK_ERR_ALIGNMENT = 6
HAWK_ERR_SCRATCH_LIMIT = 7

HAWK_DTYPE_BF16 = 0
HAWK_DTYPE_F32 = 1

_c_void_p = ctypes.c_void_p
_c_int = ctypes.c_int
_c_size_t = ctypes.c_size_t

# name -> (restype, argtypes); mirrors include/hawk_hip.h one to one
SIGNATURES = {
    "hawk_version": (_c_int, []),
    "hawk_status_string": (ctypes.c_char_p, [_c_int]),
    "hawk_scan_workspace_bytes": (_c_size_t, [_c_int] * 4),
    "hawk_scan_workspace_init": (_c_int, [_c_void_p, _c_size_t, _c_void_p]),
    "hawk_scan_workspace_status": (_c_int, [_c_void_p, _c_void_p, ctypes.POINTER(_c_int)]),
    "hawk_rglru_scan_fwd": (_c_int, [_c_void_p] * 5 + [_c_int] * 4 + [_c_void_p, _c_size_t, _c_void_p]),
    "hawk_rglru_scan_fwd_static": (_c_int, [_c_void_p] * 5 + [_c_int] * 4 + [_c_void_p]),
    "hawk_rglru_scan_fwd_static_bytes": (_c_size_t, [_c_int] * 4),
    "hawk_rglru_scan_bwd": (_c_int, [_c_void_p] * 10 + [_c_int] * 4 + [_c_void_p, _c_size_t, _c_void_p]),
    "hawk_rglru_scan_fwd_mixed": (_c_int, [_c_void_p] * 5 + [_c_int] * 5 + [_c_void_p, _c_size_t, _c_void_p]),
    "hawk_rglru_scan_bwd_mixed": (_c_int, [_c_void_p] * 10 + [_c_int] * 5 + [_c_void_p, _c_size_t, _c_void_p]),
    "hawk_rglru_scan_gated_fwd": (
        _c_int,
        [_c_void_p] * 5 + [ctypes.c_longlong] + [_c_void_p] * 3 + [_c_int] * 5 + [_c_void_p, _c_size_t, _c_void_p],
    ),
    "hawk_rglru_scan_gated_bwd": (
        _c_int,
        [_c_void_p] * 5 + [ctypes.c_longlong] + [_c_void_p] * 6 + [ctypes.c_longlong] + [_c_void_p]
        + [_c_int] * 5 + [_c_void_p, _c_size_t, _c_void_p],
    ),
    "hawk_conv1d_fwd": (_c_int, [_c_void_p] * 5 + [_c_int] * 6 + [_c_void_p]),
    "hawk_conv1d_bwd_workspace_bytes": (_c_size_t, [_c_int] * 4),
    "hawk_conv1d_bwd": (_c_int, [_c_void_p] * 6 + [_c_int] * 6 + [_c_void_p, _c_size_t, _c_void_p]),
    "hawk_conv1d_fwd_strided": (
        _c_int, [_c_void_p, ctypes.c_longlong] + [_c_void_p] * 4 + [ctypes.c_longlong] + [_c_int] * 6 + [_c_void_p]
    ),
    "hawk_conv1d_bwd_strided": (
        _c_int,
        [_c_void_p] * 2 + [ctypes.c_longlong] + [_c_void_p] * 2 + [ctypes.c_longlong] + [_c_void_p] * 2
        + [_c_int] * 6 + [_c_void_p, _c_size_t, _c_void_p],
    ),
    "hawk_conv1d_step": (_c_int, [_c_void_p] * 5 + [_c_int] * 5 + [_c_void_p]),
    "hawk_rglru_step": (_c_int, [_c_void_p] * 6 + [_c_int] * 4 + [_c_void_p]),
    "hawk_stream_capture_id": (_c_int, [_c_void_p, ctypes.POINTER(ctypes.c_ulonglong)]),
    "hawk_gate_proj_supported": (_c_int, [_c_int, _c_int]),
    "hawk_decode_core_supported": (_c_int, [_c_int] * 3),
    "hawk_decode_core_step": (
        _c_int,
        [_c_void_p] * 2 + [ctypes.c_longlong] + [_c_void_p] * 8 + [ctypes.c_longlong] + [_c_void_p] * 2
        + [_c_int] * 7 + [_c_void_p],
    ),
    "hawk_decode_core_workspace_bytes": (_c_size_t, [_c_int] * 3),
    "hawk_decode_core_step_ws": (
        _c_int,
        [_c_void_p] * 2 + [ctypes.c_longlong] + [_c_void_p] * 8 + [ctypes.c_longlong] + [_c_void_p] * 2
        + [_c_int] * 7 + [_c_void_p, _c_size_t, _c_void_p],
    ),
    "hawk_gate_proj_fwd": (_c_int, [_c_void_p] * 7 + [_c_int] * 6 + [_c_void_p]),
    "hawk_conv_gate_proj_fwd": (
        _c_int, [_c_void_p, ctypes.c_longlong] + [_c_void_p] * 9 + [_c_int] * 6 + [_c_void_p]
    ),
    "hawk_gate_proj_bwd_input": (_c_int, [_c_void_p] * 6 + [_c_int] * 6 + [_c_void_p]),
    "hawk_gate_proj_bwd_weights_workspace_bytes": (_c_size_t, [_c_int] * 3),
    "hawk_gate_proj_bwd_weights": (_c_int, [_c_void_p] * 7 + [_c_int] * 5 + [_c_void_p, _c_size_t, _c_void_p]),
    "hawk_rglru_step_gated": (
        _c_int, [_c_void_p] * 7 + [ctypes.c_longlong] + [_c_void_p] * 3 + [_c_int] * 4 + [_c_void_p]
    ),
    "hawk_stream_probe": (_c_int, [_c_void_p, _c_int, _c_void_p, _c_int, _c_size_t, _c_size_t, _c_int, _c_void_p]),
    "hawk_gate_weights_to_bf16": (_c_int, [_c_void_p] * 4 + [_c_int] * 2 + [_c_void_p]),
    "hawk_block_core_fwd": (
        _c_int, [_c_void_p, ctypes.c_longlong] + [_c_void_p] * 6 + [_c_int] + [_c_void_p] * 8 + [_c_int] * 5
        + [_c_void_p, _c_size_t, _c_void_p]
    ),
    "hawk_block_core_bwd": (
        _c_int, [_c_void_p, ctypes.c_longlong] + [_c_void_p] * 7 + [_c_int] + [_c_void_p] * 3 + [ctypes.c_longlong]
        + [_c_void_p] * 10 + [_c_int] * 5 + [_c_void_p, _c_size_t] * 3 + [_c_void_p]
    ),
}


class HawkHipError(RuntimeError):
    """A libhawk_hip entry point returned a non-zero hawk_status."""

    def __init__(self, fn: str, status: int, message: str):
        super().__init__(f"{fn} failed with status {status}: {message}")
        self.status = status


_lib = None
_lock = threading.Lock()


def load() -> ctypes.CDLL:
    """Load libhawk_hip.so, building it first only if no built library is present."""
    global _lib
    with _lock:
        if _lib is not None:
            return _lib
        if not os.path.exists(LIB_PATH):
            from .csrc.build import build

            build(force=False)
        lib = ctypes.CDLL(LIB_PATH)
        for name, (restype, argtypes) in SIGNATURES.items():
            fn = getattr(lib, name)  # AttributeError here means header and library disagree
            fn.restype = restype
            fn.argtypes = argtypes
        _lib = lib
        return lib


def status_string(status: int) -> str:
    return load().hawk_status_string(status).decode()


def check(fn: str, status: int) -> None:
    if status != HAWK_OK:
        raise HawkHipError(fn, status, status_string(status))


def dtype_code(dt: torch.dtype) -> int:
    if dt == torch.bfloat16:
        return HAWK_DTYPE_BF16
    if dt == torch.float32:
        return HAWK_DTYPE_F32
    raise TypeError(f"libhawk_hip supports bfloat16 and float32 activations, got {dt}")


def require_cuda(*tensors: torch.Tensor) -> torch.device:
    """All tensors must live on one GPU; returns that device.  There is no CPU path."""
    dev = tensors[0].device
    for t in tensors:
        if t.device.type != "cuda":
            raise RuntimeError(
                "hawk_pytorch_amd kernels run on an AMD GPU only; got a tensor on "
                f"{t.device} (there is no CPU fallback)"
            )
        if t.device != dev:
            raise RuntimeError(f"tensors on different devices: {dev} and {t.device}")
    return dev


def stream_ptr(dev: torch.device) -> int:
    return torch.cuda.current_stream(dev).cuda_stream


def ptr(t):
    return None if t is None else t.data_ptr()


def dense16(t: torch.Tensor) -> torch.Tensor:
    """Contiguous and 16-byte aligned view or copy of t (the kernels use vector loads)."""
    if not t.is_contiguous():
        t = t.contiguous()
    if t.data_ptr() % 16 != 0:
        t = t.clone(memory_format=torch.contiguous_format)
    return t


# ---------------------------------------------------------------------------------------
# Placement of the activation tensors this package allocates.  On MI355X the position of an
# address among the memory channels repeats every 1 KiB.  When the row pitch of a [B,T,D] tensor
# is a multiple of that (bf16: D a multiple of 512), every row of a 256-byte column sits at the
# same position, and tensors whose base addresses are equal modulo 1 KiB (torch's allocator
# hands out large blocks on 2 MiB boundaries) put the same column of all of them there too: a
# workgroup that streams one column tile of several tensors then keeps a quarter of the channels
# busy.  Bases 256 bytes further on from one tensor to the next (modulo 1 KiB) put the columns of
# four tensors side by side over all of them: 1-2 % on the scan kernels and on a whole block
# step at D = 2560.  The cost is 1 KiB per tensor; tensors under 16 MiB are left alone.
# HAWK_STAGGER_BYTES=0 switches it off (plain torch.empty).
# ---------------------------------------------------------------------------------------
_STAGGER_PERIOD = 1024
_STAGGER_MIN_BYTES = 16 << 20   # smaller tensors stream from the caches, and a host-bound step feels every call
_stagger_count = itertools.count()


def _stagger_bytes() -> int:
    step = int(os.environ.get("HAWK_STAGGER_BYTES", "256"))
    if step % 16 != 0 or step < 0:
        raise ValueError("HAWK_STAGGER_BYTES must be a non-negative multiple of 16")
    return step


def activation_empty(shape, dtype: torch.dtype, device) -> torch.Tensor:
    """torch.empty(shape) whose base address follows the previous call's by HAWK_STAGGER_BYTES
    modulo 1 KiB (tensors of 16 MiB and more; smaller ones are a plain torch.empty).
    Contiguous; a view of a private buffer 1 KiB larger than the tensor."""
    shape = tuple(shape)
    n = math.prod(shape)
    esz = dtype.itemsize
    if n * esz < _STAGGER_MIN_BYTES:
        return torch.empty(shape, dtype=dtype, device=device)
    step = _stagger_bytes()
    if step == 0:
        return torch.empty(shape, dtype=dtype, device=device)
    buf = torch.empty(n + _STAGGER_PERIOD // esz, dtype=dtype, device=device)
    want = (next(_stagger_count) * step) % _STAGGER_PERIOD
    off = ((want - buf.data_ptr()) % _STAGGER_PERIOD) // esz
    return buf[off:off + n].view(shape)


# ---------------------------------------------------------------------------------------
# Scan workspace: one zero-initialised buffer per (device, stream), grown on demand.
# Scans that share a workspace must be ordered on one stream, hence the key.
# ---------------------------------------------------------------------------------------
_workspaces: dict = {}
# Workspaces handed to launches recorded into HIP graphs: (device index, stream, capture id) ->
# tensors.  They belong to the graph's memory pool; a reference is kept so that their
# carry-timeout flag can be read after a replay.  All scans recorded into one capture on one
# stream share one buffer (a second, larger one only if a later scan needs more), so a captured
# training step holds one workspace, not one per layer and direction.  At most _MAX_CAPTURED
# captures are remembered (oldest dropped first; their memory stays with the graph's pool).
_captured: dict = {}
_MAX_CAPTURED = 256


def _device_index(dev: torch.device) -> int:
    return dev.index if dev.index is not None else torch.cuda.current_device()


def scan_workspace(dev: torch.device, nbytes: int) -> torch.Tensor:
    if torch.cuda.is_current_stream_capturing():
        # Captured launches get a workspace from the graph's own memory pool, zeroed by a fill
        # kernel that is part of the graph: the graph then depends on no buffer that eager code
        # or another graph also uses, whatever stream it is replayed on and in whatever order
        # graphs are replayed.  (A cached buffer created during a capture would hold nothing
        # until that one graph had been replayed.)  The scans of one capture are ordered on their
        # stream, every launch re-arms the control word and tags its carry words with its own
        # epoch, so they share the buffer as eager launches on a stream do.
        key = (_device_index(dev), stream_ptr(dev), _capture_id(dev))
        with _lock:
            held = _captured.setdefault(key, [])
            if held and held[-1].numel() >= nbytes:
                return held[-1]
        ws = torch.zeros(max(nbytes, 1 << 20), dtype=torch.uint8, device=dev)
        with _lock:
            held.append(ws)
            while len(_captured) > _MAX_CAPTURED:
                _captured.pop(next(iter(_captured)))
        return ws
    key = (_device_index(dev), stream_ptr(dev))
    with _lock:
        ws = _workspaces.get(key)
        if ws is None or ws.numel() < nbytes:
            ws = torch.zeros(max(nbytes, 1 << 20), dtype=torch.uint8, device=dev)
            _workspaces[key] = ws
    return ws


_decode_workspaces: dict = {}
_decode_captured: dict = {}   # (device, stream, capture id) -> counters of launches recorded into that graph


def _capture_id(dev: torch.device) -> int:
    cid = ctypes.c_ulonglong(0)
    with torch.cuda.device(dev):
        check("hawk_stream_capture_id", load().hawk_stream_capture_id(stream_ptr(dev), ctypes.byref(cid)))
    return cid.value


def decode_workspace(dev: torch.device, nbytes: int) -> torch.Tensor:
    """Zeroed counters for hawk_decode_core_step_ws, one buffer per (device, stream); every call
    leaves them zero, so all layers and steps on a stream share it.  Launches recorded into a HIP
    graph get one buffer per (device, stream, capture) from the graph's own memory, zeroed by one
    fill kernel that is part of the graph."""
    if torch.cuda.is_current_stream_capturing():
        key = (_device_index(dev), stream_ptr(dev), _capture_id(dev))
        with _lock:
            ws = _decode_captured.get(key)
            if ws is None or ws.numel() < nbytes:
                ws = torch.zeros(max(nbytes, 4096), dtype=torch.uint8, device=dev)
                _decode_captured[key] = ws
                while len(_decode_captured) > _MAX_CAPTURED:
                    _decode_captured.pop(next(iter(_decode_captured)))
        return ws
    key = (_device_index(dev), stream_ptr(dev))
    with _lock:
        ws = _decode_workspaces.get(key)
        if ws is None or ws.numel() < nbytes:
            ws = torch.zeros(max(nbytes, 4096), dtype=torch.uint8, device=dev)
            _decode_workspaces[key] = ws
    return ws


def release_workspaces() -> None:
    """Drop every cached scan and decode workspace (they are re-created on demand)."""
    with _lock:
        _workspaces.clear()
        _captured.clear()
        _decode_workspaces.clear()
        _decode_captured.clear()


def _flag_of(ws: torch.Tensor, dev: torch.device) -> int:
    flag = ctypes.c_int(0)
    with torch.cuda.device(dev):
        check("hawk_scan_workspace_status",
              load().hawk_scan_workspace_status(ws.data_ptr(), stream_ptr(dev), ctypes.byref(flag)))
    return flag.value


def scan_workspace_status(dev: torch.device) -> int:
    """Synchronising check of the carry-timeout flag of the current stream's workspace."""
    with _lock:
        ws = _workspaces.get((_device_index(dev), stream_ptr(dev)))
    return 0 if ws is None else _flag_of(ws, dev)


def check_scan_status(device=None) -> None:
    """Raise HawkHipError if any scan launched through this package on `device` (default: the
    current one) gave up waiting for a carry, in which case that launch's results are wrong.

    The kernels bound their wait so that a lost carry cannot hang the GPU; this is the call that
    turns such an event into an error.  It synchronises the device, so call it where the program
    synchronises anyway (end of a training step, after a graph replay, before results are used).
    Covers the cached workspaces of every stream and those of launches captured into HIP graphs.
    """
    dev = torch.device("cuda", torch.cuda.current_device()) if device is None else torch.device(device)
    idx = _device_index(dev)
    with _lock:
        todo = [ws for (d, _s), ws in _workspaces.items() if d == idx]
        todo += [ws for (d, _s, _c), held in _captured.items() if d == idx for ws in held]
    torch.cuda.synchronize(dev)
    for ws in todo:
        if _flag_of(ws, dev) != 0:
            raise HawkHipError("hawk_scan_workspace_status", HAWK_ERR_WORKSPACE,
                               "a scan tile gave up waiting for its carry: the results of that launch are "
                               "invalid; call release_workspaces() before the next scan")
