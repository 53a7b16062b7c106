"""The recurrent core of a block as one call per direction (hawk_block_core_fwd / _bwd) against
the single entry points it is made of, through the C ABI: every output bit for bit.  The single
entry points have their own parity tests against the oracle; what is pinned here is that the
shared launches (one rounding of both gates' weights, one closing reduction for dLambda, the
conv's and the projections' weight gradients) change nothing, and one case is also checked against
the oracle end to end."""

import numpy as np
import pytest
import torch

import oracle
import capi
from conftest import max_rel

pytestmark = pytest.mark.gpu


def _inputs(B, T, D, nb, w_dtype, seed, W=4):
    rng = np.random.default_rng(seed)
    bw = D // nb
    xy = capi.to_dev(rng.standard_normal((B, T, 2 * D)), "bf16")
    cw = capi.to_dev(rng.standard_normal((W, D)) * 0.5, "f32")
    cb = capi.to_dev(rng.standard_normal(D) * 0.1, "f32")
    wi = capi.to_dev(rng.standard_normal((nb, bw, bw)) / np.sqrt(bw), w_dtype)
    wa = capi.to_dev(rng.standard_normal((nb, bw, bw)) / np.sqrt(bw), w_dtype)
    bi, ba = capi.to_dev(rng.standard_normal(D) * 0.1, "f32"), capi.to_dev(rng.standard_normal(D) * 0.1, "f32")
    u = rng.uniform(0.9, 0.999, D)
    lam = capi.to_dev(np.log(u ** (-1.0 / 8.0) - 1.0), "f32")   # a^8 spread over [0.9, 0.999]
    gout = capi.to_dev(rng.standard_normal((B, T, D)), "bf16")
    return xy, cw, cb, wi, bi, wa, ba, lam, gout


def _single_calls(xy, cw, cb, wi, bi, wa, ba, lam, gout, round_weights):
    B, T, D2 = xy.shape
    D = D2 // 2
    nb = wi.shape[0]
    if round_weights and wi.dtype == torch.float32:
        wi, wa = wi.to(torch.bfloat16), wa.to(torch.bfloat16)
    x, y = xy[..., :D], xy[..., D:]
    u, xg, ag = capi.conv_gate_proj_fwd(x, cw, cb, wi, bi, wa, ba)
    out, h, h_last = capi.scan_gated_fwd(u, xg, ag, lam, y)
    d_xy = torch.full_like(xy, float("nan"))
    du, dxg, dag, dlam, _ = capi.scan_gated_bwd(u, xg, ag, lam, y, h, gout, dy=d_xy[..., D:])
    M = B * T
    capi.gate_proj_bwd_input(dxg.reshape(M, D), dag.reshape(M, D), wi, wa, torch.bfloat16, addend=du.reshape(M, D),
                             in_place=True)
    dcw, dcb = capi.conv_bwd_strided(du, x, cw, d_xy[..., :D])
    dwi, dbi, dwa, dba = capi.gate_proj_bwd_weights(u.reshape(M, D), dxg.reshape(M, D), dag.reshape(M, D), nb)
    return dict(out=out, u=u, xg=xg, ag=ag, h=h, h_last=h_last, d_xy=d_xy, dcw=dcw, dcb=dcb, dwi=dwi, dbi=dbi,
                dwa=dwa, dba=dba, dlam=dlam, du=du, w16=(wi, wa))


def _one_call_each_way(xy, cw, cb, wi, bi, wa, ba, lam, gout, round_weights):
    out, u, xg, ag, h, h_last, w16 = capi.block_core_fwd(xy, cw, cb, wi, bi, wa, ba, lam, round_weights=round_weights)
    bwi, bwa = (w16[0], w16[1]) if w16 is not None else (wi, wa)
    d_xy, dcw, dcb, dwi, dbi, dwa, dba, dlam, du = capi.block_core_bwd(xy, u, xg, ag, h, cw, bwi, bwa, lam, gout)
    return dict(out=out, u=u, xg=xg, ag=ag, h=h, h_last=h_last, d_xy=d_xy, dcw=dcw, dcb=dcb, dwi=dwi, dbi=dbi,
                dwa=dwa, dba=dba, dlam=dlam, du=du, w16=(bwi, bwa))


def _same_bits(B, T, D, nb, w_dtype, round_weights, seed):
    args = _inputs(B, T, D, nb, w_dtype, seed)
    ref = _single_calls(*args, round_weights)
    got = _one_call_each_way(*args, round_weights)
    torch.cuda.synchronize()
    for k, r in ref.items():
        if k == "w16":
            assert torch.equal(got[k][0], r[0]) and torch.equal(got[k][1], r[1]), (k, B, T, D, nb)
        else:
            assert torch.equal(got[k], r), (k, B, T, D, nb)
    return args, got


@pytest.mark.parametrize("B,T,D,nb", [(1, 32, 256, 1), (2, 33, 256, 1), (3, 100, 512, 4), (2, 77, 2560, 10),
                                      (5, 45, 96, 3), (1, 4096, 512, 16), (4, 300, 768, 3)])
@pytest.mark.parametrize("w_dtype,round_weights", [("f32", True), ("f32", False), ("bf16", True)])
def test_one_call_gives_the_bits_of_the_single_calls(B, T, D, nb, w_dtype, round_weights):
    _same_bits(B, T, D, nb, w_dtype, round_weights, seed=B * 1000 + T)


def test_benchmark_shape_and_twice_on_one_workspace():
    args, first = _same_bits(8, 4096, 2560, 10, "f32", True, seed=5)
    again = _one_call_each_way(*args, True)
    torch.cuda.synchronize()
    for k in ("out", "d_xy", "dwi", "dwa", "dbi", "dba", "dcw", "dcb", "dlam"):
        assert torch.equal(first[k], again[k]), k


def test_against_the_oracle_end_to_end():
    B, T, D, nb = 2, 160, 512, 2
    xy, cw, cb, wi, bi, wa, ba, lam, gout = _inputs(B, T, D, nb, "bf16", seed=3)
    got = _one_call_each_way(xy, cw, cb, wi, bi, wa, ba, lam, gout, True)
    f = capi.to_np
    x, y = f(xy[..., :D]), f(xy[..., D:])
    u = oracle.conv1d_fwd(x, f(cw), f(cb))
    assert max_rel(f(got["u"]), u) < 2e-2
    # from the kernel's own (bf16) intermediate values on, so that one stage's rounding is not
    # counted against the next
    u16 = f(got["u"])
    xg = oracle.block_diagonal_linear(u16.reshape(B * T, D), f(wi), f(bi).reshape(nb, -1)).reshape(B, T, D)
    ag = oracle.block_diagonal_linear(u16.reshape(B * T, D), f(wa), f(ba).reshape(nb, -1)).reshape(B, T, D)
    assert max_rel(f(got["xg"]), xg) < 2e-2 and max_rel(f(got["ag"]), ag) < 2e-2
    h = oracle.rglru_scan_fwd(u16, f(got["xg"]), f(got["ag"]), f(lam))
    assert max_rel(f(got["h"]), h) < 2e-2
    assert max_rel(f(got["out"]), oracle.gelu(y) * f(got["h"])) < 2e-2
    assert torch.equal(got["h_last"], got["h"][:, -1])


def test_rounding_of_both_weight_tensors_is_torchs():
    rng = np.random.default_rng(9)
    wi = capi.to_dev(rng.standard_normal((10, 256, 256)) * 3.0, "f32")
    wa = capi.to_dev(rng.standard_normal((10, 256, 256)) * 1e-3, "f32")
    wi.view(-1)[:4] = torch.tensor([0.0, -0.0, float("inf"), 1.00390625], device="cuda")   # the last one is a tie
    oi, oa = capi.gate_weights_to_bf16(wi, wa)
    assert torch.equal(oi, wi.to(torch.bfloat16)) and torch.equal(oa, wa.to(torch.bfloat16))
    wi, wa = (capi.to_dev(rng.standard_normal((3, 4, 4)), "f32") for _ in range(2))
    oi, oa = capi.gate_weights_to_bf16(wi, wa)
    assert torch.equal(oi, wi.to(torch.bfloat16)) and torch.equal(oa, wa.to(torch.bfloat16))


def test_refuses_what_it_does_not_serve():
    args = list(_inputs(1, 16, 256, 1, "bf16", seed=1))
    with pytest.raises(Exception, match="status 2"):
        capi.block_core_fwd(*args[:8])                       # T < 32
    args = list(_inputs(1, 64, 256, 1, "bf16", seed=1, W=3))
    with pytest.raises(Exception, match="status 2"):
        capi.block_core_fwd(*args[:8])                       # conv width 3


def test_backward_without_bias_gradients_and_with_misaligned_weight_gradients():
    """db_i / db_a may be NULL; weight-gradient tensors that do not start on 16 bytes take the
    element-by-element reduction and get the same bits."""
    args = _inputs(2, 96, 512, 2, "bf16", seed=8)
    xy, cw, cb, wi, bi, wa, ba, lam, gout = args
    out, u, xg, ag, h, _, _ = capi.block_core_fwd(xy, cw, cb, wi, bi, wa, ba, lam)
    ref = capi.block_core_bwd(xy, u, xg, ag, h, cw, wi, wa, lam, gout)
    nob = capi.block_core_bwd(xy, u, xg, ag, h, cw, wi, wa, lam, gout, with_bias=False)
    torch.cuda.synchronize()
    assert nob[4] is None and nob[6] is None
    for k in (0, 1, 2, 3, 5, 7):
        assert torch.equal(ref[k], nob[k]), k
    # the single entry point with dw tensors 4 bytes off a 16-byte boundary
    from hawk_pytorch_amd import _lib
    lib = _lib.load()
    B, T, D2 = xy.shape
    D, nb, bw, M = D2 // 2, 2, 256, B * T
    du, dxg, dag, _, _ = capi.scan_gated_bwd(u, xg, ag, lam, xy[..., D:], h, gout)
    buf = torch.zeros(2 * nb * bw * bw + 2 * D + 16, dtype=torch.float32, device="cuda")
    dwi = buf[1:1 + nb * bw * bw]
    dwa = buf[1 + nb * bw * bw:1 + 2 * nb * bw * bw]
    dbi = buf[1 + 2 * nb * bw * bw:1 + 2 * nb * bw * bw + D]
    dba = buf[1 + 2 * nb * bw * bw + D:1 + 2 * nb * bw * bw + 2 * D]
    assert dwi.data_ptr() % 16 == 4
    n = lib.hawk_gate_proj_bwd_weights_workspace_bytes(M, D, nb)
    ws = torch.empty(n, dtype=torch.uint8, device="cuda")
    code = _lib.HAWK_DTYPE_BF16
    _lib.check("bwd_weights", lib.hawk_gate_proj_bwd_weights(
        u.data_ptr(), dxg.data_ptr(), dag.data_ptr(), dwi.data_ptr(), dbi.data_ptr(), dwa.data_ptr(), dba.data_ptr(),
        M, D, nb, code, code, ws.data_ptr(), n, torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()
    assert torch.equal(dwi.view(nb, bw, bw), ref[3]) and torch.equal(dwa.view(nb, bw, bw), ref[5])
    assert torch.equal(dbi, ref[4]) and torch.equal(dba, ref[6])
