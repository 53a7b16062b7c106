"""Tensors larger than 4 GiB: every byte offset inside the kernels has to be 64-bit.

Each case replicates one slab of random data along the batch (or row) axis until a single
operand passes 2^32 bytes, runs the entry point on the whole thing, and compares every replica
bit for bit with replica 0 and with the same entry point run on the one slab alone (well below
2^31 bytes).  The kernels treat batch rows independently and deterministically, so any
difference is an address that wrapped.  (The scans fold the carries of a launch with few
independent chains in wider groups, so against the single slab they are allowed the last bit
of a bf16 value; replicas of one launch must still agree exactly.)
"""

import numpy as np
import pytest
import torch

import capi

pytestmark = pytest.mark.gpu

B, T, D = 16, 65536, 2560  # 2.68e9 elements: 5.4 GB in bf16
NB = 10


def _replicated(slab):
    big = slab.expand(B, *slab.shape[1:]).contiguous()
    assert big.numel() * big.element_size() > 2**32
    return big


def _assert_all_replicas_equal(big, one, name, exact=True):
    if exact:
        assert torch.equal(big[0], one[0]), name
    else:
        a, b = big[0].float(), one[0].float()
        assert float(((a - b).abs() / (b.abs() + 1e-3)).max()) <= 2.0**-7, name
    for b in range(1, B):
        assert torch.equal(big[b], big[0]), (name, b)


@pytest.fixture(scope="module")
def slab():
    g = torch.Generator(device="cuda").manual_seed(11)
    x, xg, ag, gout, y = (torch.randn(1, T, D, device="cuda", generator=g).to(torch.bfloat16) for _ in range(5))
    rng = np.random.default_rng(11)
    lam = capi.to_dev(np.log(np.power(rng.uniform(0.9, 0.999, size=D), -1.0 / 8.0) - 1.0), "f32")
    return x, xg, ag, gout, y, lam


def test_scan_forward_and_backward_past_4gib(slab):
    x, xg, ag, gout, _, lam = slab
    h1 = capi.scan_fwd(x, xg, ag, lam)
    g1 = capi.scan_bwd(x, xg, ag, lam, h1, gout)
    X, XG, AG, GO = (_replicated(t) for t in (x, xg, ag, gout))
    ws = capi.new_workspace(B, T, D, "bf16")
    H = capi.scan_fwd(X, XG, AG, lam, ws)
    torch.cuda.synchronize()
    _assert_all_replicas_equal(H, h1, "h", exact=False)
    G = capi.scan_bwd(X, XG, AG, lam, H, GO, ws)
    torch.cuda.synchronize()
    assert capi.workspace_flag(ws) == 0
    for name, big, one in zip(("dx", "dx_rg_lru", "da_rg_lru"), G, g1):
        _assert_all_replicas_equal(big, one, name, exact=False)
    # dLambda sums over the batch: B equal contributions (fp32 sums in a different order)
    assert float((G[3] - g1[3] * B).abs().max()) < 1e-4 * float(g1[3].abs().max()) * B


def test_gated_scan_past_4gib(slab):
    x, xg, ag, gout, y, lam = slab
    out1, h1, last1 = capi.scan_gated_fwd(x, xg, ag, lam, y)
    g1 = capi.scan_gated_bwd(x, xg, ag, lam, y, h1, gout)
    X, XG, AG, GO, Y = (_replicated(t) for t in (x, xg, ag, gout, y))
    ws = capi.new_workspace(B, T, D, "bf16")
    OUT, H, LAST = capi.scan_gated_fwd(X, XG, AG, lam, Y, ws=ws)
    torch.cuda.synchronize()
    _assert_all_replicas_equal(OUT, out1, "out", exact=False)
    _assert_all_replicas_equal(H, h1, "h", exact=False)
    _assert_all_replicas_equal(LAST, last1, "h_last", exact=False)
    del OUT
    G = capi.scan_gated_bwd(X, XG, AG, lam, Y, H, GO, ws=ws)
    torch.cuda.synchronize()
    assert capi.workspace_flag(ws) == 0
    for name, big, one in zip(("dx", "dx_rg_lru", "da_rg_lru"), G[:3], g1[:3]):
        _assert_all_replicas_equal(big, one, name, exact=False)
    _assert_all_replicas_equal(G[4], g1[4], "dy", exact=False)


def test_conv1d_past_4gib(slab):
    x, _, _, gout, _, _ = slab
    g = torch.Generator(device="cuda").manual_seed(12)
    w = torch.randn(4, D, device="cuda", generator=g)
    bias = torch.randn(D, device="cuda", generator=g)
    y1 = capi.conv_fwd(x, w, bias)
    dx1, dw1, db1 = capi.conv_bwd(gout, x, w)
    X, GO = _replicated(x), _replicated(gout)
    Y = capi.conv_fwd(X, w, bias)
    torch.cuda.synchronize()
    _assert_all_replicas_equal(Y, y1, "y")
    del Y
    DX, DW, DB = capi.conv_bwd(GO, X, w)
    torch.cuda.synchronize()
    _assert_all_replicas_equal(DX, dx1, "dx")
    # reductions over batch and time: B equal contributions, summed in a different order
    for big, one in ((DW, dw1), (DB, db1)):
        assert float((big - one * B).abs().max()) < 1e-4 * float(one.abs().max()) * B


def test_gate_projections_past_4gib(slab):
    x, xg, ag, _, _, _ = slab
    bw = D // NB
    g = torch.Generator(device="cuda").manual_seed(13)
    wi = torch.randn(NB, bw, bw, device="cuda", generator=g) / bw**0.5
    wa = torch.randn(NB, bw, bw, device="cuda", generator=g) / bw**0.5
    bi = torch.randn(D, device="cuda", generator=g)
    ba = torch.randn(D, device="cuda", generator=g)
    rows = lambda t: t.reshape(-1, D)  # noqa: E731
    oi1, oa1 = capi.gate_proj_fwd(rows(x), wi, bi, wa, ba)
    dx1 = capi.gate_proj_bwd_input(rows(xg), rows(ag), wi, wa)
    X, XG, AG = (_replicated(t) for t in (x, xg, ag))
    OI, OA = capi.gate_proj_fwd(rows(X), wi, bi, wa, ba)
    torch.cuda.synchronize()
    _assert_all_replicas_equal(OI.view(B, T, D), oi1.view(1, T, D), "x_rg_lru")
    _assert_all_replicas_equal(OA.view(B, T, D), oa1.view(1, T, D), "a_rg_lru")
    del OI, OA
    DX = capi.gate_proj_bwd_input(rows(XG), rows(AG), wi, wa)
    torch.cuda.synchronize()
    _assert_all_replicas_equal(DX.view(B, T, D), dx1.view(1, T, D), "dx")
    del DX
    # weight gradients: the replicated problem is B times the single slab
    dwi1, dbi1, dwa1, dba1 = capi.gate_proj_bwd_weights(rows(x), rows(xg), rows(ag), NB)
    DWI, DBI, DWA, DBA = capi.gate_proj_bwd_weights(rows(X), rows(XG), rows(AG), NB)
    torch.cuda.synchronize()
    for big, one in ((DWI, dwi1), (DBI, dbi1), (DWA, dwa1), (DBA, dba1)):
        scale = float(one.abs().max()) * B
        assert float((big - one * B).abs().max()) < 1e-3 * scale
