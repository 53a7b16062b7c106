"""hawk_rglru_scan_fwd_static, the forward scan that allocates nothing: its carry words live
in a fixed array inside the library's device code instead of a caller-owned workspace.

It runs the same kernels as hawk_rglru_scan_fwd, so the two must agree bit for bit (which is
stricter than the benchmark's tolerances: max-rel 1e-4 for fp32, 2e-2 for bf16), also on a
second call with a smaller input that finds the first call's words still in the array.  The
first result is also checked against the fp64 oracle.
"""

import ctypes

import numpy as np
import pytest
import torch

import oracle
import capi
from conftest import TOL, make_scan_inputs, max_rel
from hawk_pytorch_amd import _lib

pytestmark = pytest.mark.gpu


def _static_fwd(x, xg, ag, lam, h=None):
    B, T, D = x.shape
    if h is None:
        h = torch.full_like(x, float("nan"))
    rc = _lib.load().hawk_rglru_scan_fwd_static(
        x.data_ptr(), xg.data_ptr(), ag.data_ptr(), lam.data_ptr(), h.data_ptr(), B, T, D,
        _lib.dtype_code(x.dtype), torch.cuda.current_stream().cuda_stream)
    _lib.check("hawk_rglru_scan_fwd_static", rc)
    return h


def _static_flag():
    flag = ctypes.c_int(-1)
    rc = _lib.load().hawk_scan_workspace_status(None, torch.cuda.current_stream().cuda_stream, ctypes.byref(flag))
    _lib.check("hawk_scan_workspace_status", rc)
    return flag.value


def _inputs(B, T, D, dtype, seed):
    x, xg, ag, lam, _ = make_scan_inputs(B, T, D, seed=seed)
    return [capi.to_dev(a, dtype) for a in (x, xg, ag)] + [capi.to_dev(lam, "f32")]


@pytest.mark.parametrize("dtype", ["bf16", "f32"])
def test_static_scan_matches_the_workspace_scan_on_two_calls_in_a_row(dtype):
    # many time tiles and several channel tiles, then a smaller problem on the same array
    shapes = [(3, 2000, 320), (2, 700, 192)]
    for k, (B, T, D) in enumerate(shapes):
        print(f"static scan {dtype} B={B} T={T} D={D} seed {k}", flush=True)
        x, xg, ag, lam = _inputs(B, T, D, dtype, seed=k)
        want = capi.scan_fwd(x, xg, ag, lam)
        got = torch.full_like(x, float("nan"))
        before = torch.cuda.memory_allocated(), torch.cuda.memory_reserved()
        _static_fwd(x, xg, ag, lam, got)
        torch.cuda.synchronize()
        assert (torch.cuda.memory_allocated(), torch.cuda.memory_reserved()) == before
        assert _static_flag() == 0
        assert torch.equal(got.view(torch.uint8), want.view(torch.uint8)), (dtype, B, T, D)
        if k == 0:
            ref = oracle.rglru_scan_fwd(*(capi.to_np(t) for t in (x, xg, ag, lam)))
            assert max_rel(capi.to_np(got), ref) < TOL[dtype]


def test_static_scan_repeated_on_one_input_is_bitwise_stable():
    x, xg, ag, lam = _inputs(2, 1500, 256, "bf16", seed=7)
    first = _static_fwd(x, xg, ag, lam)
    for _ in range(5):
        again = _static_fwd(x, xg, ag, lam)
        assert torch.equal(again.view(torch.int16), first.view(torch.int16))
    assert _static_flag() == 0


def test_static_scan_refuses_shapes_beyond_its_array():
    # ceil(T/128) * B * D * 24 bytes: 64 * 8 * 2560 * 24 = 31.5 MB > 16 MiB
    B, T, D = 8, 8192, 2560
    x = torch.zeros((B, T, D), dtype=torch.bfloat16, device="cuda")
    lam = torch.zeros(D, dtype=torch.float32, device="cuda")
    h = torch.empty_like(x)
    rc = _lib.load().hawk_rglru_scan_fwd_static(
        x.data_ptr(), x.data_ptr(), x.data_ptr(), lam.data_ptr(), h.data_ptr(), B, T, D,
        _lib.HAWK_DTYPE_BF16, torch.cuda.current_stream().cuda_stream)
    assert rc == _lib.HAWK_ERR_SCRATCH_LIMIT
    assert "scratch" in _lib.status_string(rc)


def test_static_scan_at_the_exact_limit_of_its_array():
    """The size query is the limit: the longest chain whose words fit runs and matches the
    workspace scan; one tile more is refused."""
    lib = _lib.load()
    B, D = 1, 64
    fits, over = 10922 * 128, 10923 * 128
    assert lib.hawk_rglru_scan_fwd_static_bytes(B, fits, D, _lib.HAWK_DTYPE_BF16) <= 16 << 20
    assert lib.hawk_rglru_scan_fwd_static_bytes(B, over, D, _lib.HAWK_DTYPE_BF16) > 16 << 20
    g = torch.Generator(device="cuda").manual_seed(5)
    x, xg, ag = (torch.randn((B, over, D), generator=g, device="cuda").to(torch.bfloat16) for _ in range(3))
    lam = capi.to_dev(np.random.default_rng(5).uniform(-7.0, -2.0, D), "f32")
    h = torch.empty_like(x)
    rc = lib.hawk_rglru_scan_fwd_static(x.data_ptr(), xg.data_ptr(), ag.data_ptr(), lam.data_ptr(), h.data_ptr(),
                                        B, over, D, _lib.HAWK_DTYPE_BF16, torch.cuda.current_stream().cuda_stream)
    assert rc == _lib.HAWK_ERR_SCRATCH_LIMIT
    xs, xgs, ags = (t[:, :fits].contiguous() for t in (x, xg, ag))
    print(f"static scan at the limit B={B} T={fits} D={D}", flush=True)
    got = _static_fwd(xs, xgs, ags, lam)
    want = capi.scan_fwd(xs, xgs, ags, lam)
    torch.cuda.synchronize()
    assert _static_flag() == 0
    assert torch.equal(got.view(torch.int16), want.view(torch.int16))


def test_static_scan_at_the_benchmark_shape_fits_and_matches():
    B, T, D = 8, 4096, 2560
    g = torch.Generator(device="cuda").manual_seed(3)
    x, xg, ag = (torch.randn((B, T, D), generator=g, device="cuda").to(torch.bfloat16) for _ in range(3))
    lam = capi.to_dev(np.random.default_rng(3).uniform(-7.0, -2.0, D), "f32")
    want = capi.scan_fwd(x, xg, ag, lam)
    got = _static_fwd(x, xg, ag, lam)
    torch.cuda.synchronize()
    assert _static_flag() == 0
    assert torch.equal(got.view(torch.int16), want.view(torch.int16))
