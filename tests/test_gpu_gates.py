"""GPU parity of the fused block-diagonal gate projections (matrix-core kernels) against the
fp64 oracle, through the C ABI.  The kernels round activations and weights to bf16 and
accumulate in fp32, so the oracle is fed the bf16-rounded operands and the tolerance is the
bf16 one (2e-2 max-rel) for bf16 outputs and 1e-4 for fp32 outputs."""

import numpy as np
import pytest
import torch

import oracle
import capi
from conftest import max_rel

pytestmark = pytest.mark.gpu


def _bf16_round(a):
    return torch.from_numpy(np.asarray(a, dtype=np.float32)).to(torch.bfloat16).double().numpy()


def _case(M, D, nb, x_dtype, w_dtype, out_dtype, seed=0, bias=True):
    rng = np.random.default_rng(seed)
    bw = D // nb
    x = rng.standard_normal((M, D))
    wi = rng.standard_normal((nb, bw, bw)) / np.sqrt(bw)
    wa = rng.standard_normal((nb, bw, bw)) / np.sqrt(bw)
    bi = rng.standard_normal(D) if bias else None
    ba = rng.standard_normal(D) if bias else None
    xd = capi.to_dev(x, x_dtype)
    wid, wad = capi.to_dev(wi, w_dtype), capi.to_dev(wa, w_dtype)
    bid = capi.to_dev(bi, "f32") if bias else None
    bad = capi.to_dev(ba, "f32") if bias else None
    oi, oa = capi.gate_proj_fwd(xd, wid, bid, wad, bad, capi.TORCH_DTYPE[out_dtype])
    torch.cuda.synchronize()
    xr = _bf16_round(capi.to_np(xd))
    ref_i = oracle.block_diagonal_linear(xr, _bf16_round(capi.to_np(wid)), capi.to_np(bid) if bias else None)
    ref_a = oracle.block_diagonal_linear(xr, _bf16_round(capi.to_np(wad)), capi.to_np(bad) if bias else None)
    tol = 2e-2 if out_dtype == "bf16" else 1e-4
    assert max_rel(capi.to_np(oi), ref_i) < tol, ("x_rg_lru", M, D, nb, max_rel(capi.to_np(oi), ref_i))
    assert max_rel(capi.to_np(oa), ref_a) < tol, ("a_rg_lru", M, D, nb, max_rel(capi.to_np(oa), ref_a))
    return oi, oa


@pytest.mark.parametrize("D,nb", [(256, 1), (2560, 10), (512, 16), (512, 8), (512, 4), (768, 3), (384, 3), (96, 3)])
@pytest.mark.parametrize("M", [1, 31, 32, 33, 1000])
def test_block_widths_and_ragged_rows(M, D, nb):
    _case(M, D, nb, "bf16", "f32", "f32", seed=M + D)


@pytest.mark.parametrize("x_dtype,w_dtype,out_dtype", [("bf16", "bf16", "bf16"), ("f32", "f32", "f32"),
                                                       ("f32", "f32", "bf16"), ("bf16", "f32", "bf16")])
def test_dtype_combinations(x_dtype, w_dtype, out_dtype):
    _case(4096 + 17, 2560, 10, x_dtype, w_dtype, out_dtype, seed=3)
    _case(300, 512, 16, x_dtype, w_dtype, out_dtype, seed=4, bias=False)


def test_each_output_depends_only_on_its_own_block():
    """Perturbing the inputs of one block must leave every other block's logits bit-identical."""
    M, D, nb = 200, 1024, 8
    rng = np.random.default_rng(5)
    x = capi.to_dev(rng.standard_normal((M, D)), "bf16")
    w = [capi.to_dev(rng.standard_normal((nb, 128, 128)) / 11.0, "f32") for _ in range(2)]
    a0, b0 = capi.gate_proj_fwd(x, w[0], None, w[1], None)
    x2 = x.clone()
    x2[:, 3 * 128:4 * 128] += 1.0
    a1, b1 = capi.gate_proj_fwd(x2, w[0], None, w[1], None)
    keep = [c for c in range(D) if not 3 * 128 <= c < 4 * 128]
    assert torch.equal(a0[:, keep], a1[:, keep]) and torch.equal(b0[:, keep], b1[:, keep])
    assert not torch.equal(a0[:, 3 * 128:4 * 128], a1[:, 3 * 128:4 * 128])


@pytest.mark.parametrize("D,nb", [(2560, 10), (512, 16), (768, 6)])
@pytest.mark.parametrize("x_dtype,w_dtype,out_dtype", [("bf16", "bf16", "bf16"), ("f32", "f32", "f32"),
                                                       ("bf16", "f32", "bf16")])
def test_few_rows_and_many_rows_give_the_same_bits(D, nb, x_dtype, w_dtype, out_dtype):
    """Up to 512 rows the forward runs a kernel cut by output columns (decode), above that the
    one cut by rows; both add the same products in the same order, so the first rows of a
    600-row call must equal a call on those rows alone, bit for bit, for every small M."""
    rng = np.random.default_rng(17)
    bw = D // nb
    x = capi.to_dev(rng.standard_normal((600, D)), x_dtype)
    wi = capi.to_dev(rng.standard_normal((nb, bw, bw)) / np.sqrt(bw), w_dtype)
    wa = capi.to_dev(rng.standard_normal((nb, bw, bw)) / np.sqrt(bw), w_dtype)
    bi, ba = capi.to_dev(rng.standard_normal(D), "f32"), capi.to_dev(rng.standard_normal(D), "f32")
    big_i, big_a = capi.gate_proj_fwd(x, wi, bi, wa, ba, capi.TORCH_DTYPE[out_dtype])
    for M in (1, 7, 32, 33, 256, 300, 512):
        oi, oa = capi.gate_proj_fwd(x[:M].contiguous(), wi, bi, wa, ba, capi.TORCH_DTYPE[out_dtype])
        assert torch.equal(oi, big_i[:M]) and torch.equal(oa, big_a[:M]), M


def test_unsupported_shapes_are_refused():
    from hawk_pytorch_amd import _lib
    lib = _lib.load()
    assert lib.hawk_gate_proj_supported(2560, 10) == 1 and lib.hawk_gate_proj_supported(512, 16) == 1
    assert lib.hawk_gate_proj_supported(2560, 3) == 0 and lib.hawk_gate_proj_supported(1024, 2) == 0
    x = torch.zeros((4, 1024), device="cuda")
    w = torch.zeros((2, 512, 512), device="cuda")
    with pytest.raises(_lib.HawkHipError):
        capi.gate_proj_fwd(x, w, None, w, None)


def test_full_benchmark_shape_against_the_library_gemm():
    """B*T = 32768 tokens, D = 2560, 10 blocks: every element against torch's batched GEMM
    on the same bf16 operands (fp32 accumulation on both sides)."""
    M, D, nb = 32768, 2560, 10
    g = torch.Generator(device="cuda").manual_seed(1)
    x = torch.randn((M, D), generator=g, device="cuda").to(torch.bfloat16)
    wi = torch.randn((nb, 256, 256), generator=g, device="cuda") / 16.0
    wa = torch.randn((nb, 256, 256), generator=g, device="cuda") / 16.0
    bi = torch.randn(D, generator=g, device="cuda")
    ba = torch.randn(D, generator=g, device="cuda")
    oi, oa = capi.gate_proj_fwd(x, wi, bi, wa, ba, torch.float32)
    xb = x.reshape(M, nb, 256).transpose(0, 1)
    for got, w, b in ((oi, wi, bi), (oa, wa, ba)):
        ref = torch.bmm(xb.float(), w.to(torch.bfloat16).float()).transpose(0, 1).reshape(M, D) + b
        err = float((got - ref).abs().max() / ref.abs().max())
        assert err < 1e-4, err


# ---------------------------------------------------------------------------------------- input gradient
def _bwd_input_case(M, D, nb, g_dtype, w_dtype, dx_dtype, seed=0):
    rng = np.random.default_rng(seed)
    bw = D // nb
    gi, ga = rng.standard_normal((M, D)), rng.standard_normal((M, D))
    wi = rng.standard_normal((nb, bw, bw)) / np.sqrt(bw)
    wa = rng.standard_normal((nb, bw, bw)) / np.sqrt(bw)
    gid, gad = capi.to_dev(gi, g_dtype), capi.to_dev(ga, g_dtype)
    wid, wad = capi.to_dev(wi, w_dtype), capi.to_dev(wa, w_dtype)
    dx = capi.gate_proj_bwd_input(gid, gad, wid, wad, capi.TORCH_DTYPE[dx_dtype])
    torch.cuda.synchronize()
    zeros = np.zeros((M, D))
    ref = (oracle.block_diagonal_linear_bwd(zeros, _bf16_round(capi.to_np(wid)), _bf16_round(capi.to_np(gid)))[0]
           + oracle.block_diagonal_linear_bwd(zeros, _bf16_round(capi.to_np(wad)), _bf16_round(capi.to_np(gad)))[0])
    tol = 2e-2 if dx_dtype == "bf16" else 1e-4
    assert max_rel(capi.to_np(dx), ref) < tol, (M, D, nb, max_rel(capi.to_np(dx), ref))


@pytest.mark.parametrize("D,nb", [(256, 1), (2560, 10), (512, 16), (512, 8), (512, 4), (768, 3), (384, 3), (96, 3)])
@pytest.mark.parametrize("M", [1, 33, 1000])
def test_input_gradient_block_widths_and_ragged_rows(M, D, nb):
    _bwd_input_case(M, D, nb, "bf16", "f32", "f32", seed=M + D)


@pytest.mark.parametrize("g_dtype,w_dtype,dx_dtype", [("bf16", "bf16", "bf16"), ("f32", "f32", "f32"),
                                                      ("bf16", "f32", "bf16"), ("f32", "bf16", "bf16")])
def test_input_gradient_dtype_combinations(g_dtype, w_dtype, dx_dtype):
    _bwd_input_case(4096 + 17, 2560, 10, g_dtype, w_dtype, dx_dtype, seed=7)
    _bwd_input_case(300, 512, 16, g_dtype, w_dtype, dx_dtype, seed=8)


def test_input_gradient_is_the_adjoint_of_the_forward():
    """<forward(x), (gi, ga)> == <x, bwd_input(gi, ga)> with zero bias, on the full shape."""
    M, D, nb = 32768, 2560, 10
    g = torch.Generator(device="cuda").manual_seed(2)
    mk = lambda: torch.randn((M, D), generator=g, device="cuda").to(torch.bfloat16)  # noqa: E731
    x, gi, ga = mk(), mk(), mk()
    wi = torch.randn((nb, 256, 256), generator=g, device="cuda") / 16.0
    wa = torch.randn((nb, 256, 256), generator=g, device="cuda") / 16.0
    oi, oa = capi.gate_proj_fwd(x, wi, None, wa, None, torch.float32)
    dx = capi.gate_proj_bwd_input(gi, ga, wi, wa, torch.float32)
    lhs = (oi.double() * gi.double()).sum() + (oa.double() * ga.double()).sum()
    rhs = (x.double() * dx.double()).sum()
    assert abs(float(lhs - rhs)) < 1e-5 * abs(float(lhs)), (float(lhs), float(rhs))


# ---------------------------------------------------------------------------------------- weight gradients
def _bwd_weights_case(M, D, nb, x_dtype, g_dtype, seed=0):
    rng = np.random.default_rng(seed)
    bw = D // nb
    x, gi, ga = (rng.standard_normal((M, D)) for _ in range(3))
    xd, gid, gad = capi.to_dev(x, x_dtype), capi.to_dev(gi, g_dtype), capi.to_dev(ga, g_dtype)
    dwi, dbi, dwa, dba = capi.gate_proj_bwd_weights(xd, gid, gad, nb)
    torch.cuda.synchronize()
    xr = _bf16_round(capi.to_np(xd))
    zeros_w = np.zeros((nb, bw, bw))
    for name, gd, dw, db in (("i", gid, dwi, dbi), ("a", gad, dwa, dba)):
        gr = _bf16_round(capi.to_np(gd))
        _, ref_w, ref_b = oracle.block_diagonal_linear_bwd(xr, zeros_w, gr)
        assert max_rel(capi.to_np(dw), ref_w) < 1e-4, (name, M, D, nb, max_rel(capi.to_np(dw), ref_w))
        assert max_rel(capi.to_np(db), ref_b.reshape(-1)) < 1e-4, (name, "bias", M, D, nb)


@pytest.mark.parametrize("D,nb", [(256, 1), (2560, 10), (512, 16), (512, 8), (512, 4), (768, 3), (384, 3), (96, 3)])
@pytest.mark.parametrize("M", [1, 33, 1000])
def test_weight_gradients_block_widths_and_ragged_rows(M, D, nb):
    _bwd_weights_case(M, D, nb, "bf16", "bf16", seed=M + D)


@pytest.mark.parametrize("x_dtype,g_dtype", [("f32", "f32"), ("bf16", "f32"), ("f32", "bf16")])
def test_weight_gradients_dtype_combinations(x_dtype, g_dtype):
    _bwd_weights_case(4096 + 17, 2560, 10, x_dtype, g_dtype, seed=9)
    _bwd_weights_case(300, 512, 16, x_dtype, g_dtype, seed=10)


def test_weight_gradients_full_shape_against_the_library_gemm_and_reproducible():
    M, D, nb = 32768, 2560, 10
    g = torch.Generator(device="cuda").manual_seed(3)
    mk = lambda: torch.randn((M, D), generator=g, device="cuda").to(torch.bfloat16)  # noqa: E731
    x, gi, ga = mk(), mk(), mk()
    first = capi.gate_proj_bwd_weights(x, gi, ga, nb)
    second = capi.gate_proj_bwd_weights(x, gi, ga, nb)
    for a, b in zip(first, second):
        assert torch.equal(a, b)
    xb = x.reshape(M, nb, 256).transpose(0, 1).float()
    for gd, dw, db in ((gi, first[0], first[1]), (ga, first[2], first[3])):
        ref_w = torch.bmm(xb.transpose(1, 2), gd.reshape(M, nb, 256).transpose(0, 1).float())
        assert float((dw - ref_w).abs().max() / ref_w.abs().max()) < 1e-4
        ref_b = gd.double().sum(dim=0)
        assert float((db.double() - ref_b).abs().max() / ref_b.abs().max()) < 1e-4


def test_input_gradient_adds_the_addend_also_in_place():
    M, D, nb = 1000, 2560, 10
    g = torch.Generator(device="cuda").manual_seed(4)
    mk = lambda: torch.randn((M, D), generator=g, device="cuda").to(torch.bfloat16)  # noqa: E731
    gi, ga, add = mk(), mk(), mk()
    wi = torch.randn((nb, 256, 256), generator=g, device="cuda") / 16.0
    wa = torch.randn((nb, 256, 256), generator=g, device="cuda") / 16.0
    plain = capi.gate_proj_bwd_input(gi, ga, wi, wa, torch.float32)
    want = plain + add.float()
    got = capi.gate_proj_bwd_input(gi, ga, wi, wa, torch.bfloat16, addend=add)
    assert max_rel(capi.to_np(got), capi.to_np(want)) < 2e-2
    got32 = capi.gate_proj_bwd_input(gi, ga, wi, wa, torch.float32, addend=add.float())
    assert max_rel(capi.to_np(got32), capi.to_np(want)) < 1e-6
    buf = add.clone()
    same = capi.gate_proj_bwd_input(gi, ga, wi, wa, torch.bfloat16, addend=buf, in_place=True)
    assert same.data_ptr() == buf.data_ptr() and torch.equal(buf, got)


# ---------------------------------------------------------------------------------------
# The forward with the temporal conv in front: same bits as the two separate calls.
# ---------------------------------------------------------------------------------------
def _conv_gate_case(B, T, D, nb, w_dtype, strided, seed):
    rng = np.random.default_rng(seed)
    bw = D // nb
    xy = capi.to_dev(rng.standard_normal((B, T, 2 * D if strided else D)), "bf16")
    x = xy[..., :D]
    cw = capi.to_dev(rng.standard_normal((4, D)) * 0.5, "f32")
    cb = capi.to_dev(rng.standard_normal(D) * 0.1, "f32")
    wi = capi.to_dev(rng.standard_normal((nb, bw, bw)) / np.sqrt(bw), w_dtype)
    wa = capi.to_dev(rng.standard_normal((nb, bw, bw)) / np.sqrt(bw), w_dtype)
    bi, ba = capi.to_dev(rng.standard_normal(D), "f32"), capi.to_dev(rng.standard_normal(D), "f32")
    u, oi, oa = capi.conv_gate_proj_fwd(x, cw, cb, wi, bi, wa, ba)
    u_ref = capi.conv_fwd(x.contiguous(), cw, cb, y_dtype=torch.bfloat16)
    oi_ref, oa_ref = capi.gate_proj_fwd(u_ref.reshape(B * T, D), wi, bi, wa, ba, torch.bfloat16)
    torch.cuda.synchronize()
    assert torch.equal(u, u_ref), ("conv output", B, T, D, nb)
    assert torch.equal(oi.reshape(B * T, D), oi_ref), ("x_rg_lru", B, T, D, nb)
    assert torch.equal(oa.reshape(B * T, D), oa_ref), ("a_rg_lru", B, T, D, nb)
    # and the conv itself against the oracle (the separate kernel has its own tests; this pins
    # the masking of rows before each sequence's first one)
    ref = oracle.conv1d_fwd(capi.to_np(x).astype(np.float64), capi.to_np(cw).astype(np.float64),
                            capi.to_np(cb).astype(np.float64))
    assert max_rel(capi.to_np(u), ref) < 2e-2


@pytest.mark.parametrize("B,T,D,nb", [(1, 32, 256, 1), (2, 33, 256, 1), (3, 100, 512, 4), (2, 77, 2560, 10),
                                      (5, 45, 96, 3), (1, 4096, 512, 16), (4, 64, 768, 3), (7, 37, 384, 3)])
@pytest.mark.parametrize("strided", [False, True])
def test_conv_in_front_gives_the_bits_of_the_two_calls(B, T, D, nb, strided):
    _conv_gate_case(B, T, D, nb, "bf16", strided, seed=B * 1000 + T)


def test_conv_in_front_with_fp32_weights_and_many_tiles_per_workgroup():
    _conv_gate_case(8, 1111, 2560, 10, "f32", True, seed=11)
    _conv_gate_case(2, 4096 + 5, 1024, 4, "f32", False, seed=12)


def test_conv_in_front_refuses_what_it_does_not_serve():
    x = torch.zeros(1, 16, 256, dtype=torch.bfloat16, device="cuda")
    cw, cb = torch.zeros(4, 256, device="cuda"), torch.zeros(256, device="cuda")
    w = torch.zeros(1, 256, 256, dtype=torch.bfloat16, device="cuda")
    with pytest.raises(Exception, match="status 2"):
        capi.conv_gate_proj_fwd(x, cw, cb, w, None, w, None)                      # T < 32
    x = torch.zeros(1, 64, 256, dtype=torch.bfloat16, device="cuda")
    with pytest.raises(Exception, match="status 2"):
        capi.conv_gate_proj_fwd(x, torch.zeros(3, 256, device="cuda"), cb, w, None, w, None)   # width 3
