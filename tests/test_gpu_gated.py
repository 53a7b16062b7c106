"""GPU parity of the scan fused with the block's gate, out = gelu(y) * h, against the fp64
oracle, through the C ABI.  Tolerances as for the plain scan: max-rel 1e-4 (fp32), 2e-2
(bf16 activations / state)."""

import numpy as np
import pytest
import torch

import oracle
import capi
from conftest import TOL, make_scan_inputs, max_rel

pytestmark = pytest.mark.gpu

GRADS = ("dx", "dx_rg_lru", "da_rg_lru", "da_param", "dy")


def _gate_input(B, T, D, dtype, seed, layout):
    """y as the model produces it: `half` = second half of a [B,T,2D] projection (row stride
    2D), `dense` = its own tensor, `odd` = rows D+3 apart (forces one channel per lane)."""
    rng = np.random.default_rng(seed + 77)
    y = 1.5 * rng.standard_normal((B, T, D))
    y.flat[:: 7] *= 3.0  # some entries deep in both GELU tails
    if layout == "dense":
        yd = capi.to_dev(y, dtype)
    else:
        ld = 2 * D if layout == "half" else (D + 3 if D % 2 == 0 else D + 4)  # "odd": an odd row stride
        wide = torch.zeros((B, T, ld), dtype=capi.TORCH_DTYPE[dtype], device="cuda")
        yd = wide[..., ld - D:] if layout == "half" else wide[..., :D]
        yd.copy_(capi.to_dev(y, dtype))
    return yd, capi.to_np(yd)


def _run(B, T, D, in_dtype, state_dtype, layout="half", seed=0, lo=0.9, hi=0.999, ws=None, want_h=True):
    x, xg, ag, lam, gout = make_scan_inputs(B, T, D, seed=seed, lo=lo, hi=hi)
    xd, xgd, agd = (capi.to_dev(a, in_dtype) for a in (x, xg, ag))
    x, xg, ag = (capi.to_np(t) for t in (xd, xgd, agd))
    god = capi.to_dev(gout, state_dtype)
    gout = capi.to_np(god)
    lam_d = capi.to_dev(lam, "f32")
    lam = capi.to_np(lam_d)
    yd, y = _gate_input(B, T, D, state_dtype, seed, layout)
    tol = TOL["bf16" if "bf16" in (in_dtype, state_dtype) else "f32"]

    out_d, h_d, hl_d = capi.scan_gated_fwd(xd, xgd, agd, lam_d, yd, capi.TORCH_DTYPE[state_dtype], want_h=want_h, ws=ws)
    torch.cuda.synchronize()
    h_ref, out_ref = oracle.rglru_scan_gated_fwd(x, xg, ag, lam, y)
    assert max_rel(capi.to_np(out_d), out_ref) < tol, ("out", max_rel(capi.to_np(out_d), out_ref))
    assert max_rel(capi.to_np(hl_d), h_ref[:, -1, :]) < tol, "h_last"
    if not want_h:
        return
    h_gpu = capi.to_np(h_d)
    assert max_rel(h_gpu, h_ref) < tol, "h"
    # the plain entry point gives the same h up to the last bit (its time tiles are longer, so
    # the fp32 carries are rounded at different places)
    h_plain = capi.scan_fwd_mixed(xd, xgd, agd, lam_d, capi.TORCH_DTYPE[state_dtype])
    assert max_rel(capi.to_np(h_plain), h_gpu) <= (2.0 ** -7 if state_dtype == "bf16" else 2e-6)

    got = capi.scan_gated_bwd(xd, xgd, agd, lam_d, yd, h_d, god, ws=ws)
    torch.cuda.synchronize()
    ref = oracle.rglru_scan_gated_bwd(x, xg, ag, lam, y, h_gpu, gout)
    for name, g, r in zip(GRADS, got, ref):
        g = capi.to_np(g)
        assert np.all(np.isfinite(g)), name
        assert max_rel(g, r) < tol, (name, B, T, D, in_dtype, state_dtype, layout, max_rel(g, r))


@pytest.mark.parametrize("dtypes", [("f32", "f32"), ("bf16", "bf16"), ("f32", "bf16")])
@pytest.mark.parametrize("layout", ["half", "dense", "odd"])
def test_config0_shape(dtypes, layout):
    _run(1, 256, 512, *dtypes, layout=layout)


@pytest.mark.parametrize("dtypes", [("f32", "f32"), ("bf16", "bf16"), ("f32", "bf16")])
@pytest.mark.parametrize("T", [1, 2, 3, 63, 64, 65, 79, 80, 81, 95, 96, 97, 128, 129, 200, 257, 1000])
def test_time_lengths_around_tile_edges(T, dtypes):
    _run(2, T, 128, *dtypes, seed=T)


@pytest.mark.parametrize("dtypes", [("f32", "f32"), ("bf16", "bf16")])
@pytest.mark.parametrize("T", [1, 63, 65, 100, 129, 200])
def test_time_lengths_around_tile_edges_with_many_chains(T, dtypes):
    """The 64-row backward tiles that launches with 128 or more chains take (8 x 2048 channels)."""
    _run(8, T, 2048, *dtypes, seed=400 + T)


@pytest.mark.parametrize("dtypes", [("f32", "f32"), ("bf16", "bf16")])
@pytest.mark.parametrize("D", [1, 2, 3, 64, 66, 130, 320, 1000])
def test_channel_counts_including_ragged_tiles(D, dtypes):
    _run(2, 131, D, *dtypes, layout="dense" if D < 8 else "half", seed=D)


@pytest.mark.parametrize("dtypes", [("f32", "f32"), ("bf16", "bf16")])
def test_many_tiles_long_memory(dtypes):
    _run(1, 8192, 128, *dtypes, lo=0.99, hi=0.9999, seed=5)


def test_forward_without_the_state_sequence():
    _run(2, 700, 192, "bf16", "bf16", want_h=False)
    _run(2, 700, 192, "f32", "f32", want_h=False)


def test_gate_gradient_can_land_in_a_wider_buffer():
    B, T, D = 2, 300, 128
    x, xg, ag, lam, gout = make_scan_inputs(B, T, D, seed=3)
    dev = [capi.to_dev(a, "bf16") for a in (x, xg, ag, gout)]
    lam_d = capi.to_dev(lam, "f32")
    wide = torch.randn((B, T, 2 * D), device="cuda").to(torch.bfloat16)
    y = wide[..., D:]
    out, h, _ = capi.scan_gated_fwd(dev[0], dev[1], dev[2], lam_d, y)
    grad_wide = torch.full((B, T, 2 * D), 7.0, dtype=torch.bfloat16, device="cuda")
    dense = capi.scan_gated_bwd(dev[0], dev[1], dev[2], lam_d, y, h, dev[3])
    strided = capi.scan_gated_bwd(dev[0], dev[1], dev[2], lam_d, y, h, dev[3], dy=grad_wide[..., D:])
    torch.cuda.synchronize()
    for a, b in zip(dense, strided):
        assert torch.equal(a, b.contiguous())
    assert torch.all(grad_wide[..., :D] == 7.0)  # the other half is untouched


def test_gate_extremes_stay_finite():
    B, T, D = 1, 200, 64
    x, xg, ag, lam, gout = make_scan_inputs(B, T, D, seed=9)
    for dtype in ("f32", "bf16"):
        dev = [capi.to_dev(a, dtype) for a in (x, xg, ag, gout)]
        lam_d = capi.to_dev(lam, "f32")
        y = np.zeros((B, T, D))
        y[..., 0::4] = 1e4
        y[..., 1::4] = -1e4
        y[..., 2::4] = 40.0
        y[..., 3::4] = -40.0
        yd = capi.to_dev(y, dtype)
        out, h, _ = capi.scan_gated_fwd(dev[0], dev[1], dev[2], lam_d, yd)
        got = capi.scan_gated_bwd(dev[0], dev[1], dev[2], lam_d, yd, h, dev[3])
        torch.cuda.synchronize()
        hn, on = capi.to_np(h), capi.to_np(out)
        assert np.all(np.isfinite(on))
        assert np.all(on[..., 1::2] == 0.0)  # gelu(-40) and gelu(-1e4) are zero to fp32
        assert max_rel(on[..., 0::2], (capi.to_np(yd) * hn)[..., 0::2]) < TOL[dtype]
        for g in got:
            assert np.all(np.isfinite(capi.to_np(g)))


@pytest.mark.parametrize("B,T,D", [(8, 4096, 2560), (2, 32768, 4096)])
def test_full_benchmark_shapes_bf16(B, T, D):
    """Full size: oracle on a channel subset; the fused result against the unfused kernels
    (plain scan + torch's gelu) on every element."""
    g = torch.Generator(device="cuda").manual_seed(11)
    mk = lambda: torch.randn((B, T, D), generator=g, device="cuda").to(torch.bfloat16)  # noqa: E731
    x, xg, ag, gout = mk(), mk(), mk(), mk()
    wide = torch.randn((B, T, 2 * D), generator=g, device="cuda").to(torch.bfloat16)
    y = wide[..., D:]
    u = torch.rand(D, generator=g, device="cuda") * 0.099 + 0.9
    lam = torch.log(u.double() ** (-1.0 / 8.0) - 1.0).float()
    ws = capi.new_workspace(B, T, D, "bf16")
    out, h, h_last = capi.scan_gated_fwd(x, xg, ag, lam, y, ws=ws)
    dx, dxg, dag, dlam, dy = capi.scan_gated_bwd(x, xg, ag, lam, y, h, gout, ws=ws)
    torch.cuda.synchronize()
    assert capi.workspace_flag(ws) == 0
    assert max_rel(capi.scan_fwd(x, xg, ag, lam, ws).float().cpu().numpy(), h.float().cpu().numpy()) <= 2.0 ** -7
    assert torch.equal(h_last, h[:, -1, :])
    # unfused: gradient reaching h computed by torch in fp32, rounded to bf16 like the saved tensors
    yf = y.float()
    gelu = torch.nn.functional.gelu(yf)
    ref_out = gelu * h.float()
    assert max_rel(out.float().cpu().numpy(), ref_out.cpu().numpy()) < TOL["bf16"]
    gh = (gout.float() * gelu).to(torch.bfloat16)
    ref = capi.scan_bwd(x, xg, ag, lam, h, gh, ws)
    torch.cuda.synchronize()
    for name, a, b in zip(GRADS, (dx, dxg, dag, dlam), ref):
        assert max_rel(a.float().cpu().numpy(), b.float().cpu().numpy()) < TOL["bf16"], name
    sl = slice(0, D, D // 8)
    cols = [t[..., sl].float().cpu().numpy().astype(np.float64) for t in (x, xg, ag, y, h, gout)]
    ref = oracle.rglru_scan_gated_bwd(cols[0], cols[1], cols[2], lam[sl].double().cpu().numpy(), cols[3], cols[4], cols[5])
    for name, a, r in zip(GRADS, (dx, dxg, dag, dlam, dy), ref):
        a = a[..., sl].float().cpu().numpy()
        assert max_rel(a, r) < TOL["bf16"], (name, max_rel(a, r))
