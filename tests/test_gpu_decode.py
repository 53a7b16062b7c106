"""GPU parity of the decode-step kernels and of the prefill -> decode hand-off."""

import numpy as np
import pytest
import torch

import oracle
import capi
from conftest import TOL, make_scan_inputs, max_rel

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize("B,D", [(1, 64), (1, 2560), (3, 130), (256, 2560), (5, 7)])
def test_rglru_step(B, D, dtype):
    x, xg, ag, lam, st = make_scan_inputs(B, 1, D, seed=B + D)
    d = [capi.to_dev(a[:, 0], dtype) for a in (x, xg, ag, st)]
    xr, xgr, agr, sr = (capi.to_np(t) for t in d)
    lam_d = capi.to_dev(lam, "f32")
    state = d[3].clone()
    h = capi.rglru_step(d[0], d[1], d[2], lam_d, state)
    ref = oracle.rglru_step(xr, xgr, agr, capi.to_np(lam_d), sr)
    assert max_rel(capi.to_np(h), ref) < TOL[dtype]
    assert torch.equal(state, h)  # the cache buffer now holds the new state


def test_rglru_step_bf16_cache_fp32_activations():
    """Upstream keeps the cache in bf16 while the step runs in fp32 (hawk/cache.py:12-17)."""
    B, D = 4, 256
    x, xg, ag, lam, st = make_scan_inputs(B, 1, D, seed=3)
    d = [capi.to_dev(a[:, 0], "f32") for a in (x, xg, ag)]
    state = capi.to_dev(st[:, 0], "bf16")
    sr = capi.to_np(state)
    lam_d = capi.to_dev(lam, "f32")
    h = capi.rglru_step(d[0], d[1], d[2], lam_d, state)
    ref = oracle.rglru_step(*(capi.to_np(t) for t in d), capi.to_np(lam_d), sr)
    assert max_rel(capi.to_np(h), ref) < TOL["f32"]
    assert torch.equal(state, h.to(torch.bfloat16))


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize("with_bias", [True, False])
@pytest.mark.parametrize("B,D", [(1, 64), (256, 2560), (3, 130), (5, 7)])
def test_rglru_step_gated(B, D, with_bias, dtype):
    """Biases of the two gate projections added in the kernel, state updated in place,
    gelu(y) * h returned; y is the second half of a [B, 2D] projection."""
    x, xg, ag, lam, st = make_scan_inputs(B, 1, D, seed=B + D + 1)
    rng = np.random.default_rng(B * D)
    d = [capi.to_dev(a[:, 0], dtype) for a in (x, xg, ag, st)]
    xr, xgr, agr, sr = (capi.to_np(t) for t in d)
    lam_d = capi.to_dev(lam, "f32")
    bi = capi.to_dev(rng.standard_normal(D), "f32") if with_bias else None
    ba = capi.to_dev(rng.standard_normal(D), "f32") if with_bias else None
    wide = capi.to_dev(2.0 * rng.standard_normal((B, 2 * D)), dtype)
    y = wide[:, D:]
    state = d[3].clone()
    out, h = capi.rglru_step_gated(d[0], d[1], d[2], bi, ba, lam_d, y, state)
    zero = np.zeros(D)
    h_ref = oracle.rglru_step(xr, xgr + (capi.to_np(bi) if with_bias else zero),
                              agr + (capi.to_np(ba) if with_bias else zero), capi.to_np(lam_d), sr)
    assert max_rel(capi.to_np(h), h_ref) < TOL[dtype]
    assert max_rel(capi.to_np(out), oracle.gelu(capi.to_np(y)) * h_ref) < TOL[dtype]
    assert torch.equal(state, h)
    # h_out is optional
    state2 = d[3].clone()
    out2, none = capi.rglru_step_gated(d[0], d[1], d[2], bi, ba, lam_d, y, state2, want_h=False)
    assert none is None and torch.equal(out2, out) and torch.equal(state2, state)


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize("W", [1, 2, 4, 8])
@pytest.mark.parametrize("B,D", [(1, 64), (256, 2560), (3, 30)])
def test_conv_step(B, D, W, dtype):
    rng = np.random.default_rng(B + D + W)
    st = capi.to_dev(rng.standard_normal((B, max(W - 1, 1), D))[:, : W - 1], dtype) if W > 1 else None
    xn = capi.to_dev(rng.standard_normal((B, D)), dtype)
    w = capi.to_dev(rng.standard_normal((W, D)) * 0.5, "f32")
    b = capi.to_dev(rng.standard_normal(D), "f32")
    if W == 1:
        st = torch.empty((B, 0, D), dtype=xn.dtype, device="cuda")
        st_np = np.zeros((B, 0, D))
        dummy = torch.zeros(16, device="cuda")  # a valid pointer for the unused state argument
        y = capi.conv_step(dummy, xn, w, b)
        ref_y, _ = oracle.conv1d_step(st_np, capi.to_np(xn), capi.to_np(w), capi.to_np(b))
        assert max_rel(capi.to_np(y), ref_y) < TOL[dtype]
        return
    st = st.contiguous()
    before = capi.to_np(st)
    y = capi.conv_step(st, xn, w, b)
    ref_y, ref_state = oracle.conv1d_step(before, capi.to_np(xn), capi.to_np(w), capi.to_np(b))
    assert max_rel(capi.to_np(y), ref_y) < TOL[dtype]
    assert np.array_equal(capi.to_np(st), ref_state)  # pure data movement: bit exact


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_prefill_then_steps_track_the_full_scan(dtype):
    """scan over T rows, then K single-token steps from its last state, against the scan
    over T+K rows; same for the conv with its rolling window."""
    B, T, K, D, W = 2, 200, 5, 128, 4
    x, xg, ag, lam, _ = make_scan_inputs(B, T + K, D, seed=17)
    d = [capi.to_dev(a, dtype) for a in (x, xg, ag)]
    lam_d = capi.to_dev(lam, "f32")
    h_full = capi.scan_fwd(*d, lam_d)
    h_pre = capi.scan_fwd(*(t[:, :T].contiguous() for t in d), lam_d)
    state = h_pre[:, -1].contiguous().float()  # fp32 cache: no extra rounding between steps
    for k in range(K):
        row = [t[:, T + k].contiguous() for t in d]
        h = capi.rglru_step(*row, lam_d, state)
        assert max_rel(capi.to_np(h), capi.to_np(h_full[:, T + k])) < TOL[dtype]

    rng = np.random.default_rng(4)
    w = capi.to_dev(rng.standard_normal((W, D)) * 0.5, "f32")
    b = capi.to_dev(rng.standard_normal(D), "f32")
    y_full = capi.conv_fwd(d[0], w, b)
    conv_state = d[0][:, T - (W - 1): T].contiguous()
    for k in range(K):
        y = capi.conv_step(conv_state, d[0][:, T + k].contiguous(), w, b)
        assert max_rel(capi.to_np(y), capi.to_np(y_full[:, T + k])) < TOL[dtype]


def _core_operands(B, D, nb, W, w_dtype, state_dtype, seed):
    rng = np.random.default_rng(seed)
    bw = D // nb
    wide = capi.to_dev(rng.standard_normal((B, 2 * D)), "bf16")   # the input projection: [x | y]
    conv_state = capi.to_dev(rng.standard_normal((B, W - 1, D)), "bf16")
    conv_w = capi.to_dev(rng.standard_normal((W, D)) * 0.5, "f32")
    conv_b = capi.to_dev(rng.standard_normal(D) * 0.1, "f32")
    w_i = capi.to_dev(rng.standard_normal((nb, bw, bw)) / np.sqrt(bw), w_dtype)
    w_a = capi.to_dev(rng.standard_normal((nb, bw, bw)) / np.sqrt(bw), w_dtype)
    b_i = capi.to_dev(rng.standard_normal(D), "f32")
    b_a = capi.to_dev(rng.standard_normal(D), "f32")
    lam = capi.to_dev(np.log(np.power(rng.uniform(0.9, 0.999, size=D), -1.0 / 8.0) - 1.0), "f32")
    state = capi.to_dev(rng.standard_normal((B, D)), state_dtype)
    return wide, conv_state, conv_w, conv_b, w_i, b_i, w_a, b_a, lam, state


@pytest.mark.parametrize("w_dtype,state_dtype", [("bf16", "bf16"), ("f32", "bf16"), ("bf16", "f32"), ("f32", "f32")])
@pytest.mark.parametrize("B,D,nb,W", [(256, 2560, 10, 4), (1, 2560, 10, 4), (33, 512, 16, 4), (5, 256, 4, 2),
                                      (70, 256, 2, 8), (3, 64, 2, 1), (64, 1024, 4, 4)])
def test_decode_core_step_matches_the_three_separate_launches(B, D, nb, W, w_dtype, state_dtype):
    """One launch against hawk_conv1d_step + hawk_gate_proj_fwd + hawk_rglru_step_gated on the
    same operands (x and y are the two halves of one [B, 2D] tensor): the conv window exactly,
    state and output to the last bits of their dtype, over three consecutive tokens."""
    wide, cs, conv_w, conv_b, w_i, b_i, w_a, b_a, lam, st = _core_operands(B, D, nb, W, w_dtype, state_dtype, B + D + W)
    cs_ref, st_ref = cs.clone(), st.clone()
    rng = np.random.default_rng(7)
    for step in range(3):
        x_new, y = wide[:, :D], wide[:, D:]
        out = capi.decode_core_step(cs if W > 1 else None, x_new, conv_w, conv_b, w_i, b_i, w_a, b_a, lam, y, st)
        u = capi.conv_step(cs_ref, x_new.contiguous(), conv_w, conv_b, torch.bfloat16)
        xg, ag = capi.gate_proj_fwd(u, w_i, b_i, w_a, b_a, torch.bfloat16)
        out_ref, _ = capi.rglru_step_gated(u, xg, ag, None, None, lam, y, st_ref)
        torch.cuda.synchronize()
        assert torch.equal(cs, cs_ref), step
        tol = 2.0 ** -7 if state_dtype == "bf16" else 1e-5
        assert max_rel(capi.to_np(st), capi.to_np(st_ref)) <= tol, step
        assert max_rel(capi.to_np(out), capi.to_np(out_ref)) <= 2.0 ** -7, step
        wide = capi.to_dev(rng.standard_normal((B, 2 * D)), "bf16")


def test_decode_core_step_against_the_oracle():
    """The same launch against the fp64 restatement: conv step, block-diagonal projections with
    their biases, the recurrence and the gate."""
    B, D, nb, W = 37, 512, 4, 4
    wide, cs, conv_w, conv_b, w_i, b_i, w_a, b_a, lam, st = _core_operands(B, D, nb, W, "f32", "f32", 99)
    x_new, y = wide[:, :D], wide[:, D:]
    n = capi.to_np
    u_ref, cs_next = oracle.conv1d_step(n(cs), n(x_new), n(conv_w), n(conv_b))
    xg = oracle.block_diagonal_linear(u_ref, n(w_i), n(b_i))
    ag = oracle.block_diagonal_linear(u_ref, n(w_a), n(b_a))
    h_ref = oracle.rglru_step(u_ref, xg, ag, n(lam), n(st))
    out_ref = oracle.gelu(n(y)) * h_ref
    out = capi.decode_core_step(cs, x_new, conv_w, conv_b, w_i, b_i, w_a, b_a, lam, y, st)
    assert np.array_equal(n(cs), cs_next.astype(np.float32))
    assert max_rel(n(st), h_ref) < TOL["bf16"]
    assert max_rel(n(out), out_ref) < TOL["bf16"]


@pytest.mark.parametrize("state_dtype", ["bf16", "f32"])
def test_decode_core_step_with_operands_that_forbid_16_byte_accesses(state_dtype):
    """y with an odd row stride, recc_state and out 8 bytes off a 16-byte boundary: the step
    falls back to element-wise accesses for them and gives the same result."""
    B, D, nb, W = 45, 512, 4, 4
    wide, cs, conv_w, conv_b, w_i, b_i, w_a, b_a, lam, st = _core_operands(B, D, nb, W, "bf16", state_dtype, 21)
    x_new = wide[:, :D]
    y_odd = torch.zeros(B, D + 1, dtype=torch.bfloat16, device="cuda")
    y_odd[:, :D] = wide[:, D:]
    y = y_odd[:, :D]
    assert y.stride(0) % 2 == 1
    off = 8 // st.element_size()
    st_buf = torch.zeros(B * D + off, dtype=st.dtype, device="cuda")
    st_off = st_buf[off:].view(B, D)
    st_off.copy_(st)
    assert st_off.data_ptr() % 16 == 8
    cs_ref, st_ref = cs.clone(), st.clone()
    out = capi.decode_core_step(cs, x_new, conv_w, conv_b, w_i, b_i, w_a, b_a, lam, y, st_off)
    out_ref = capi.decode_core_step(cs_ref, x_new, conv_w, conv_b, w_i, b_i, w_a, b_a, lam, wide[:, D:], st_ref)
    assert torch.equal(cs, cs_ref)
    assert torch.equal(st_off, st_ref)
    assert torch.equal(out, out_ref)


@pytest.mark.parametrize("w_dtype,state_dtype", [("bf16", "bf16"), ("f32", "f32")])
@pytest.mark.parametrize("B,D,nb,W", [(256, 2560, 10, 4), (1, 2560, 10, 4), (33, 512, 4, 4), (100, 256, 4, 2),
                                      (70, 256, 2, 8), (3, 128, 2, 1), (64, 1024, 4, 4), (700, 512, 2, 4),
                                      (40, 256, 8, 4)])
def test_decode_core_step_with_counters_is_bit_identical_to_the_one_without(B, D, nb, W, w_dtype, state_dtype):
    """hawk_decode_core_step_ws cuts a block's output columns over up to four workgroups (block
    widths of 64 and more, launches small enough to gain from it); the workgroup that is last to
    have read a conv window rolls it.  Window, state and output must equal the single-workgroup
    launch bit for bit over consecutive tokens on one workspace, which every call must leave
    holding zeros."""
    wide, cs, conv_w, conv_b, w_i, b_i, w_a, b_a, lam, st = _core_operands(B, D, nb, W, w_dtype, state_dtype, B + D + W)
    cs_ref, st_ref = cs.clone(), st.clone()
    ws = capi.decode_core_workspace(B, D, nb)
    rng = np.random.default_rng(11)
    for step in range(4):
        x_new, y = wide[:, :D], wide[:, D:]
        out = capi.decode_core_step(cs if W > 1 else None, x_new, conv_w, conv_b, w_i, b_i, w_a, b_a, lam, y, st, ws=ws)
        out_ref = capi.decode_core_step(cs_ref if W > 1 else None, x_new, conv_w, conv_b, w_i, b_i, w_a, b_a, lam, y,
                                        st_ref)
        torch.cuda.synchronize()
        assert torch.equal(cs, cs_ref), step
        assert torch.equal(st, st_ref), step
        assert torch.equal(out, out_ref), step
        assert int(ws.view(torch.int32).abs().sum()) == 0, step
        wide = capi.to_dev(rng.standard_normal((B, 2 * D)), "bf16")
