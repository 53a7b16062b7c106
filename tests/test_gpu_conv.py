"""GPU parity of the temporal conv1d kernels (forward, backward, with state) against the
fp64 oracle, through the C ABI."""

import numpy as np
import pytest
import torch

import oracle
import capi
from conftest import TOL, max_rel

pytestmark = pytest.mark.gpu


def _case(B, T, D, W, dtype, seed, y_dtype=None):
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((B, T, D))
    gy = rng.standard_normal((B, T, D))
    w = rng.standard_normal((W, D)) * 0.5  # benchmark init: N(0, 1/4)
    b = rng.standard_normal(D) * 0.1
    xd, gyd = capi.to_dev(x, dtype), capi.to_dev(gy, dtype)
    wd, bd = capi.to_dev(w, "f32"), capi.to_dev(b, "f32")
    xr, gyr, wr, br = (capi.to_np(t) for t in (xd, gyd, wd, bd))
    tol = TOL[dtype]
    yt = None if y_dtype is None else capi.TORCH_DTYPE[y_dtype]
    y = capi.conv_fwd(xd, wd, bd, y_dtype=yt)
    assert max_rel(capi.to_np(y), oracle.conv1d_fwd(xr, wr, br)) < (tol if y_dtype != "f32" else 1e-4)
    dx, dw, db = capi.conv_bwd(gyd, xd, wd)
    rdx, rdw, rdb = oracle.conv1d_bwd(gyr, xr, wr)
    assert max_rel(capi.to_np(dx), rdx) < tol
    assert max_rel(capi.to_np(dw), rdw) < 1e-4  # fp32 accumulation of exactly representable products
    assert max_rel(capi.to_np(db), rdb) < 1e-4


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize("T", [1, 2, 3, 4, 15, 16, 17, 63, 64, 65, 300, 1030])
def test_width4_time_lengths(T, dtype):
    _case(2, T, 128, 4, dtype, seed=T)


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize("D", [1, 2, 6, 64, 100, 256, 260, 1000])
def test_width4_channel_counts(D, dtype):
    _case(3, 70, D, 4, dtype, seed=D)


@pytest.mark.parametrize("W", [1, 2, 3, 5, 8])
def test_other_temporal_widths(W):
    _case(2, 50, 96, W, "f32", seed=W)
    _case(2, 50, 96, W, "bf16", seed=W)


def test_bf16_input_fp32_output_is_the_upstream_promotion():
    _case(2, 100, 128, 4, "bf16", seed=5, y_dtype="f32")


@pytest.mark.parametrize("W", [2, 4, 6])
@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_forward_with_state_equals_joined_sequence(W, dtype):
    rng = np.random.default_rng(9)
    B, T, D = 2, 40, 128
    full = capi.to_dev(rng.standard_normal((B, T + W - 1, D)), dtype)
    wd = capi.to_dev(rng.standard_normal((W, D)) * 0.5, "f32")
    bd = capi.to_dev(rng.standard_normal(D), "f32")
    y_full = capi.conv_fwd(full, wd, bd)
    y_state = capi.conv_fwd(full[:, W - 1:].contiguous(), wd, bd, state=full[:, : W - 1].contiguous())
    assert torch.equal(y_state, y_full[:, W - 1:])


def test_benchmark_shape_bf16():
    """B=8, T=4096, D=2560, bf16: oracle on a channel subset, db/dw on all channels by
    torch reductions in fp64."""
    B, T, D, W = 8, 4096, 2560, 4
    g = torch.Generator(device="cuda").manual_seed(3)
    x = torch.randn(B, T, D, device="cuda", generator=g).to(torch.bfloat16)
    gy = torch.randn(B, T, D, device="cuda", generator=g).to(torch.bfloat16)
    w = (torch.randn(W, D, device="cuda", generator=g) * 0.5).float()
    b = torch.zeros(D, device="cuda")
    y = capi.conv_fwd(x, w, b)
    dx, dw, db = capi.conv_bwd(gy, x, w)
    sel = torch.arange(0, D, 80, device="cuda")
    take = lambda t: capi.to_np(t.index_select(-1, sel))  # noqa: E731
    assert max_rel(take(y), oracle.conv1d_fwd(take(x), take(w), take(b))) < TOL["bf16"]
    rdx, rdw, rdb = oracle.conv1d_bwd(take(gy), take(x), take(w))
    assert max_rel(take(dx), rdx) < TOL["bf16"]
    assert max_rel(take(dw), rdw) < 1e-4
    assert max_rel(take(db), rdb) < 1e-4
    db_all = gy.double().sum(dim=(0, 1))
    assert max_rel(capi.to_np(db), db_all.cpu().numpy()) < 1e-4
    dw_last = (gy.double() * x.double()).sum(dim=(0, 1))  # tap on the current row is w[W-1]
    assert max_rel(capi.to_np(dw[W - 1]), dw_last.cpu().numpy()) < 1e-4


# ---------------------------------------------------------------------------------------
# Rows further apart than D: one half of a [B,T,2D] tensor read and written in place.
# ---------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize("B,T,D,W,pad", [(2, 70, 128, 4, 128), (3, 33, 260, 4, 4), (1, 200, 100, 4, 2),
                                         (2, 50, 63, 4, 1), (2, 40, 96, 3, 96), (1, 17, 64, 8, 8)])
def test_strided_rows_give_the_bits_of_the_dense_call(B, T, D, W, pad, dtype):
    rng = np.random.default_rng(B * 100 + T)
    wide = capi.to_dev(rng.standard_normal((B, T, D + pad)), dtype)
    x = wide[..., :D]
    gy = capi.to_dev(rng.standard_normal((B, T, D)), dtype)
    w, b = capi.to_dev(rng.standard_normal((W, D)) * 0.5, "f32"), capi.to_dev(rng.standard_normal(D) * 0.1, "f32")
    y_ref = capi.conv_fwd(x.contiguous(), w, b)
    dx_ref, dw_ref, db_ref = capi.conv_bwd(gy, x.contiguous(), w)
    # outputs into the first D columns of a wider tensor whose other columns must stay as they are
    out_wide = torch.full((B, T, D + pad), 7.0, dtype=x.dtype, device="cuda")
    capi.conv_fwd_strided(x, w, b, out_wide[..., :D])
    dx_wide = torch.full((B, T, D + pad), 7.0, dtype=x.dtype, device="cuda")
    dw, db = capi.conv_bwd_strided(gy, x, w, dx_wide[..., :D])
    torch.cuda.synchronize()
    assert torch.equal(out_wide[..., :D], y_ref) and bool((out_wide[..., D:] == 7.0).all())
    assert torch.equal(dx_wide[..., :D], dx_ref) and bool((dx_wide[..., D:] == 7.0).all())
    assert torch.equal(dw, dw_ref) and torch.equal(db, db_ref)


def test_strided_rows_refuse_a_stride_below_the_channel_count():
    from hawk_pytorch_amd import _lib

    x = torch.zeros(1, 8, 64, device="cuda")
    w, b = torch.zeros(4, 64, device="cuda"), torch.zeros(64, device="cuda")
    lib = _lib.load()
    rc = lib.hawk_conv1d_fwd_strided(x.data_ptr(), 32, w.data_ptr(), b.data_ptr(), None, x.data_ptr(), 64, 1, 8, 64, 4,
                                     1, 1, None)
    assert rc == _lib.HAWK_ERR_BAD_SHAPE
