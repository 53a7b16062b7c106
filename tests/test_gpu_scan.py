"""GPU parity of the RG-LRU scan kernels against the fp64 oracle, through the C ABI.

Tolerances are the benchmark's: max-rel (max |err| / max |ref| per tensor) 1e-4 for fp32
activations, 2e-2 for bf16 activations with fp32 state.  Inputs are rounded to the
activation dtype first and the oracle sees exactly the rounded values.
"""

import numpy as np
import pytest
import scipy.signal
import torch

import oracle
import capi
from conftest import TOL, make_scan_inputs, max_rel

pytestmark = pytest.mark.gpu


def _round_inputs(arrs, dtype):
    """Device tensors in `dtype` plus the fp64 numpy image of what the device holds."""
    dev = [capi.to_dev(a, dtype) for a in arrs]
    return dev, [capi.to_np(t) for t in dev]


def _run_case(B, T, D, dtype, seed=0, lo=0.9, hi=0.999, ws=None, channels=None):
    x, xg, ag, lam, gout = make_scan_inputs(B, T, D, seed=seed, lo=lo, hi=hi)
    (dx_, dxg_, dag_, dgo_), (x, xg, ag, gout) = _round_inputs((x, xg, ag, gout), dtype)
    lam_d = capi.to_dev(lam, "f32")
    lam = capi.to_np(lam_d)
    h_d = capi.scan_fwd(dx_, dxg_, dag_, lam_d, ws)
    g_d = capi.scan_bwd(dx_, dxg_, dag_, lam_d, h_d, dgo_, ws)
    torch.cuda.synchronize()
    sl = slice(None) if channels is None else channels
    h_ref = oracle.rglru_scan_fwd(x[..., sl], xg[..., sl], ag[..., sl], lam[sl])
    tol = TOL[dtype]
    h_gpu = capi.to_np(h_d)[..., sl]
    assert max_rel(h_gpu, h_ref) < tol, ("h", B, T, D, dtype, max_rel(h_gpu, h_ref))
    # the backward consumes the h the forward stored (rounded to dtype), as upstream does
    ref = oracle.rglru_scan_bwd(x[..., sl], xg[..., sl], ag[..., sl], lam[sl], h_gpu, gout[..., sl])
    names = ("dx", "dx_rg_lru", "da_rg_lru", "da_param")
    for name, got, want in zip(names, g_d, ref):
        got = capi.to_np(got)[..., sl]
        assert np.all(np.isfinite(got)), name
        assert max_rel(got, want) < tol, (name, B, T, D, dtype, max_rel(got, want))
    # and the whole fwd+bwd chain against the all-fp64 chain
    ref64 = oracle.rglru_scan_bwd(x[..., sl], xg[..., sl], ag[..., sl], lam[sl], h_ref, gout[..., sl])
    for name, got, want in zip(names, g_d, ref64):
        assert max_rel(capi.to_np(got)[..., sl], want) < tol, (name + " (fp64 chain)", B, T, D, dtype)
    return h_d, g_d


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_config0_shape(dtype):
    """B=1, T=256, D=512: the CPU-reference configuration of the benchmark definition."""
    _run_case(1, 256, 512, dtype, seed=0)


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize("T", [1, 2, 3, 7, 8, 9, 63, 64, 65, 127, 128, 129, 200, 257, 1000])
def test_time_lengths_around_tile_edges(T, dtype):
    _run_case(2, T, 128, dtype, seed=T)


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize("T", [1, 5, 63, 64, 65, 100, 129, 200])
def test_time_lengths_around_tile_edges_with_many_chains(T, dtype):
    """128 or more independent chains (batch rows x channel tiles) switch the backward to 64-row
    tiles, which keep alpha from the local pass for the replay; rows past T must stay the
    identity there too.  8 x 2048 channels: 128 chains in bf16, 256 in fp32."""
    _run_case(8, T, 2048, dtype, seed=300 + T)


@pytest.mark.parametrize("B,T,D", [(1, 9000, 128), (1, 6100, 512), (2, 5000, 512), (3, 4500, 256)])
def test_long_sequences_on_very_few_chains(B, T, D):
    """Up to 8 independent chains (batch rows x channel tiles) space the checkpoints of the carry
    chain 16 positions apart, up to 4 chains 32 apart (a wave then fetches several predecessors):
    1, 4, 8 and 6 chains here in bf16, over 36 to 71 forward positions."""
    _run_case(B, T, D, "bf16", seed=500 + D, lo=0.99, hi=0.9999)
    _run_case(B, T, D, "f32", seed=501 + D)


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize("D", [1, 2, 3, 64, 66, 128, 130, 192, 320, 1000])
def test_channel_counts_including_ragged_tiles(D, dtype):
    """The C ABI takes any D; odd D runs one channel per lane, and D that does not fill the
    last channel tile leaves lanes idle."""
    _run_case(2, 150, D, dtype, seed=100 + D)


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_many_tiles_long_memory(dtype):
    """Long-memory regime of the long-context configuration (alpha^8 in [0.99, 0.9999]) over
    many time tiles: the carry chain is what is exercised."""
    _run_case(1, 8192, 128, dtype, seed=5, lo=0.99, hi=0.9999)


@pytest.mark.parametrize("shape", [(1, 256, 512), (2, 1000, 192), (1, 1, 64), (2, 97, 65), (1, 4096, 128)])
def test_mixed_precision_entry_fp32_inputs_bf16_state(shape):
    """fp32 x / gate logits, bf16 h and grad_out, fp32 gradients: what the model feeds the
    scan under autocast.  The oracle sees the exact fp32 inputs; tolerance is the bf16 one
    because h and grad_out are bf16."""
    B, T, D = shape
    x, xg, ag, lam, gout = make_scan_inputs(B, T, D, seed=T + D)
    (dx_, dxg_, dag_), (xr, xgr, agr) = _round_inputs((x, xg, ag), "f32")
    go_d = capi.to_dev(gout, "bf16")
    gor = capi.to_np(go_d)
    lam_d = capi.to_dev(lam, "f32")
    lam_r = capi.to_np(lam_d)
    h = capi.scan_fwd_mixed(dx_, dxg_, dag_, lam_d, torch.bfloat16)
    assert h.dtype == torch.bfloat16
    h_ref = oracle.rglru_scan_fwd(xr, xgr, agr, lam_r)
    assert max_rel(capi.to_np(h), h_ref) < TOL["bf16"]
    grads = capi.scan_bwd_mixed(dx_, dxg_, dag_, lam_d, h, go_d)
    assert all(g.dtype == torch.float32 for g in grads)
    ref = oracle.rglru_scan_bwd(xr, xgr, agr, lam_r, capi.to_np(h), gor)
    for name, got, want in zip(("dx", "dx_rg_lru", "da_rg_lru", "da_param"), grads, ref):
        assert max_rel(capi.to_np(got), want) < TOL["bf16"], name
    # the mixed forward must agree with "cast inputs to bf16, then scan" up to input rounding,
    # and be closer to the exact-input oracle than that path is
    h_cast = capi.scan_fwd(dx_.bfloat16(), dxg_.bfloat16(), dag_.bfloat16(), lam_d)
    err_mixed = np.abs(capi.to_np(h) - h_ref).mean()
    err_cast = np.abs(capi.to_np(h_cast) - h_ref).mean()
    assert err_mixed <= err_cast * 1.05


def test_unsupported_dtype_pairs_are_refused():
    x = torch.zeros(1, 8, 64, device="cuda", dtype=torch.bfloat16)
    lam = torch.zeros(64, device="cuda")
    with pytest.raises(Exception, match="dtype"):
        capi.scan_fwd_mixed(x, x, x, lam, torch.float32)  # bf16 inputs with fp32 state: not offered


def test_workspace_reuse_across_shapes_and_launches():
    """One workspace serves repeated launches and smaller shapes; tags of earlier launches
    must never be taken for fresh ones."""
    ws = capi.new_workspace(2, 2048, 256, "bf16")
    first = _run_case(2, 2048, 256, "bf16", seed=1, ws=ws)
    for seed, (B, T, D) in enumerate([(2, 2048, 256), (1, 700, 128), (2, 2048, 256), (2, 65, 64)]):
        _run_case(B, T, D, "bf16", seed=seed + 1, ws=ws)
    again = _run_case(2, 2048, 256, "bf16", seed=1, ws=ws)
    assert torch.equal(first[0], again[0])
    for a, b in zip(first[1][:3], again[1][:3]):
        assert torch.equal(a, b)
    assert capi.workspace_flag(ws) == 0


def test_result_does_not_depend_on_how_time_is_tiled():
    """Chunk invariance: the first T1 rows of a long scan equal a scan of only those rows
    (a different number of tiles and a different position of every row inside its tile)."""
    x, xg, ag, lam, _ = make_scan_inputs(1, 1024, 128, seed=11, lo=0.99, hi=0.9999)
    d = [capi.to_dev(a, "f32") for a in (x, xg, ag)]
    lam_d = capi.to_dev(lam, "f32")
    h_long = capi.to_np(capi.scan_fwd(*d, lam_d))
    for T1 in (1, 50, 64, 100, 513):
        part = [t[:, :T1].contiguous() for t in d]
        h_short = capi.to_np(capi.scan_fwd(*part, lam_d))
        assert max_rel(h_short, h_long[:, :T1]) < 2e-6, T1


def test_constant_gates_equal_lfilter_on_gpu():
    rng = np.random.default_rng(3)
    B, T, D = 2, 700, 64
    x = rng.standard_normal((B, T, D))
    xg = np.broadcast_to(rng.standard_normal((1, 1, D)), (B, T, D)).copy()
    ag = np.broadcast_to(rng.standard_normal((1, 1, D)), (B, T, D)).copy()
    lam = rng.uniform(-6.0, 1.0, size=D)
    d = [capi.to_dev(a, "f32") for a in (x, xg, ag)]
    xr, xgr, agr = (capi.to_np(t) for t in d)
    lam_d = capi.to_dev(lam, "f32")
    lam_r = capi.to_np(lam_d)
    h = capi.to_np(capi.scan_fwd(*d, lam_d))
    alpha = np.exp(-8.0 / (1.0 + np.exp(-agr[0, 0])) * np.log1p(np.exp(lam_r)))
    beta = np.sqrt(1 - alpha**2) / (1.0 + np.exp(-xgr[0, 0])) * xr
    for c in range(D):
        ref = scipy.signal.lfilter([1.0], [1.0, -alpha[c]], beta[:, :, c], axis=1)
        assert max_rel(h[:, :, c], ref) < 1e-4, c


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_gate_extremes(dtype):
    x, xg, ag, lam, gout = make_scan_inputs(1, 200, 64, seed=21)
    lam_d = capi.to_dev(lam, "f32")
    # r -> 0: alpha = 1, beta = 0, h == 0 exactly; gradients stay finite
    d = [capi.to_dev(a, dtype) for a in (x, xg, np.full_like(ag, -300.0), gout)]
    h = capi.scan_fwd(d[0], d[1], d[2], lam_d)
    assert torch.all(h == 0)
    grads = capi.scan_bwd(d[0], d[1], d[2], lam_d, h, d[3])
    for g in grads:
        assert torch.all(torch.isfinite(g.float()))
    # alpha -> 0: h_t = i_t x_t
    d2 = [capi.to_dev(a, dtype) for a in (x, xg, np.full_like(ag, 60.0))]
    big = capi.to_dev(np.full_like(lam, 30.0), "f32")
    h2 = capi.to_np(capi.scan_fwd(*d2, big))
    ref = capi.to_np(d2[0]) / (1.0 + np.exp(-capi.to_np(d2[1])))
    assert max_rel(h2, ref) < TOL[dtype]
    # huge logits of both signs do not produce NaN
    wild = np.where(np.random.default_rng(2).random(ag.shape) < 0.5, -1e4, 1e4)
    d3 = [capi.to_dev(a, dtype) for a in (x, wild, -wild, gout)]
    h3 = capi.scan_fwd(d3[0], d3[1], d3[2], lam_d)
    assert torch.all(torch.isfinite(h3.float()))
    for g in capi.scan_bwd(d3[0], d3[1], d3[2], lam_d, h3, d3[3]):
        assert torch.all(torch.isfinite(g.float()))


def test_clip_branch_of_the_sqrt_derivative():
    """Lambda = -20 puts every element inside the clip (1 - alpha^2 < 2.5e-7), where the
    oracle's closed form (derivative = 1000) was pinned on the CPU."""
    x, xg, ag, _, gout = make_scan_inputs(2, 70, 64, seed=31)
    lam = np.full(64, -20.0)
    d = [capi.to_dev(a, "f32") for a in (x, xg, ag, gout)]
    xr, xgr, agr, gor = (capi.to_np(t) for t in d)
    lam_d = capi.to_dev(lam, "f32")
    h = capi.scan_fwd(d[0], d[1], d[2], lam_d)
    got = capi.scan_bwd(d[0], d[1], d[2], lam_d, h, d[3])
    want = oracle.rglru_scan_bwd(xr, xgr, agr, lam, capi.to_np(h), gor)
    for name, a, b in zip(("dx", "dxg", "dag", "dlam"), got, want):
        assert max_rel(capi.to_np(a), b) < 1e-4, name


@pytest.mark.parametrize(
    "B,T,D,lo,hi",
    [(8, 4096, 2560, 0.9, 0.999), (2, 32768, 4096, 0.99, 0.9999)],
    ids=["scan_B8_T4096_D2560", "long_context_B2_T32768_D4096"],
)
def test_full_benchmark_shapes_bf16(B, T, D, lo, hi):
    """Full benchmark sizes.  Channels are independent, so the oracle is run on a strided
    subset of channels over all of B and T; every channel is covered by two size-independent
    properties: linearity of h in x, and sum_t(gout*h)-style adjoint identity
    <gout, h(x)> == <dx, x> (h is linear in x with adjoint dx for fixed gates)."""
    rng = np.random.default_rng(7)
    lam = np.log(np.power(rng.uniform(lo, hi, size=D), -1.0 / 8.0) - 1.0)
    lam_d = capi.to_dev(lam, "f32")
    g = torch.Generator(device="cuda").manual_seed(7)
    x, xg, ag, gout = (torch.randn(B, T, D, device="cuda", generator=g).to(torch.bfloat16) for _ in range(4))
    ws = capi.new_workspace(B, T, D, "bf16")
    h = capi.scan_fwd(x, xg, ag, lam_d, ws)
    dx, dxg, dag, dlam = capi.scan_bwd(x, xg, ag, lam_d, h, gout, ws)
    torch.cuda.synchronize()
    assert capi.workspace_flag(ws) == 0

    sel = np.arange(0, D, D // 32)[:32]
    sel_t = torch.from_numpy(sel).cuda()
    take = lambda t: capi.to_np(t.index_select(2, sel_t))  # noqa: E731
    xs, xgs, ags, gos = take(x), take(xg), take(ag), take(gout)
    h_ref = oracle.rglru_scan_fwd(xs, xgs, ags, lam[sel])
    assert max_rel(take(h), h_ref) < TOL["bf16"]
    ref = oracle.rglru_scan_bwd(xs, xgs, ags, capi.to_np(lam_d)[sel], take(h), gos)
    assert max_rel(take(dx), ref[0]) < TOL["bf16"]
    assert max_rel(take(dxg), ref[1]) < TOL["bf16"]
    assert max_rel(take(dag), ref[2]) < TOL["bf16"]
    assert max_rel(capi.to_np(dlam)[sel], ref[3]) < TOL["bf16"]

    # adjoint identity over ALL channels: <gout, h> == <dx, x> up to bf16 rounding of h, dx
    lhs = (gout.float() * h.float()).sum(dim=(0, 1)).double()
    rhs = (dx.float() * x.float()).sum(dim=(0, 1)).double()
    scale = (gout.float() * h.float()).abs().sum(dim=(0, 1)).double()
    assert float(((lhs - rhs).abs() / scale).max()) < 2e-3
    # linearity over ALL channels: h(2x) == 2 h(x) exactly in bf16 (power-of-two scaling)
    h2 = capi.scan_fwd((x.float() * 2).to(torch.bfloat16), xg, ag, lam_d, ws)
    assert torch.equal(h2.float(), h.float() * 2)


@pytest.mark.parametrize("B,T,D,dtype", [
    (8, 2100, 1024, "bf16"),    # 64 chains, last tile cut short
    (8, 1000, 2560, "bf16"),    # 160 chains (the short backward tiles), few tiles in time
    (16, 1345, 1280, "bf16"),   # 160 chains, ragged
    (8, 1500, 1024, "f32"),     # one channel per lane
    (12, 1111, 960, "f32"),
])
def test_launches_of_a_thousand_tiles_and_more(B, T, D, dtype):
    """Launches with more tiles than the device holds at once (several rounds of workgroups,
    many chains in flight): full parity against the oracle, all channels."""
    _run_case(B, T, D, dtype, seed=B + T)


def test_scan_launches_replay_correctly_from_a_hip_graph():
    """Forward, backward and the gated pair captured once and replayed several times, with
    eager launches on the same workspace in between; every replay must reproduce the eager
    result bit for bit (the launch epoch lives in the workspace, not in the captured arguments)."""
    B, T, D = 2, 1500, 256
    x, xg, ag, lam, gout = make_scan_inputs(B, T, D, seed=21)
    dev = [capi.to_dev(a, "bf16") for a in (x, xg, ag, gout)]
    lam_d = capi.to_dev(lam, "f32")
    wide = torch.randn(B, T, 2 * D, device="cuda").to(torch.bfloat16)
    y = wide[..., D:]
    ws = capi.new_workspace(B, T, D, "bf16")

    def run():
        h = capi.scan_fwd(dev[0], dev[1], dev[2], lam_d, ws)
        g = capi.scan_bwd(dev[0], dev[1], dev[2], lam_d, h, dev[3], ws)
        out, hg, hl = capi.scan_gated_fwd(dev[0], dev[1], dev[2], lam_d, y, ws=ws)
        gg = capi.scan_gated_bwd(dev[0], dev[1], dev[2], lam_d, y, hg, dev[3], ws=ws)
        return (h, *g, out, hg, hl, *gg)

    eager = [t.clone() for t in run()]
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        run()
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        captured = run()
    for rep in range(4):
        for t in captured:
            t.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        for a, b in zip(captured, eager):
            assert torch.equal(a, b), rep
        again = run()  # eager launches between replays move the workspace's epoch along
        torch.cuda.synchronize()
        for a, b in zip(again, eager):
            assert torch.equal(a, b), rep
    assert capi.workspace_flag(ws) == 0


def test_two_streams_scan_concurrently_with_their_own_workspaces():
    """Two scans of the benchmark size in flight at once on two streams, each with its own
    workspace (the rule of the C ABI), several rounds: every result must equal the one obtained
    alone.  A tile only ever waits for tiles of its own launch that have already started, so
    two launches sharing the compute units cannot block each other."""
    B, T, D = 8, 4096, 2560
    g = torch.Generator(device="cuda").manual_seed(31)
    lam = capi.to_dev(np.log(np.power(np.random.default_rng(31).uniform(0.9, 0.999, size=D), -1.0 / 8.0) - 1.0), "f32")
    sets = []
    for _ in range(2):
        x, xg, ag, go = (torch.randn(B, T, D, device="cuda", generator=g).to(torch.bfloat16) for _ in range(4))
        ws = capi.new_workspace(B, T, D, "bf16")
        h = capi.scan_fwd(x, xg, ag, lam, ws)
        grads = capi.scan_bwd(x, xg, ag, lam, h, go, ws)
        sets.append((x, xg, ag, go, ws, h, grads))
    torch.cuda.synchronize()
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    for s in streams:
        s.wait_stream(torch.cuda.current_stream())
    for _ in range(3):
        got = []
        for (x, xg, ag, go, ws, _, _), s in zip(sets, streams):
            with torch.cuda.stream(s):
                h = capi.scan_fwd(x, xg, ag, lam, ws)
                got.append((h, capi.scan_bwd(x, xg, ag, lam, h, go, ws)))
        torch.cuda.synchronize()
        for (h, grads), (_, _, _, _, ws, h_ref, grads_ref) in zip(got, sets):
            assert capi.workspace_flag(ws) == 0
            assert torch.equal(h, h_ref)
            for a, b in zip(grads, grads_ref):
                assert torch.equal(a, b)


@pytest.mark.parametrize("dtype", ["bf16", "f32"])
def test_results_do_not_depend_on_where_the_tensors_start(dtype):
    """The same values in tensors whose bases are 0, 16, 48, 256 or 272 bytes apart modulo 1 KiB
    (the host code places the activations it allocates 256 bytes apart, callers may pass any
    16-byte aligned pointers): the same bits."""
    B, T, D = 3, 700, 640
    arrs = make_scan_inputs(B, T, D, seed=21)
    x, xg, ag, lam, gout = arrs
    lam_d = capi.to_dev(lam, "f32")
    n = x.size
    td = capi.TORCH_DTYPE[dtype]
    esz = 2 if dtype == "bf16" else 4

    def carve(step):
        pad = step // esz
        buf = torch.zeros(4 * (n + pad) + 2048, dtype=td, device="cuda")
        first = ((-buf.data_ptr()) % 1024) // esz
        out = []
        for i, a in enumerate((x, xg, ag, gout)):
            t = buf[first + i * (n + pad): first + i * (n + pad) + n].view(a.shape)
            t.copy_(capi.to_dev(a, dtype))
            out.append(t)
        return out, buf

    ref = None
    for step in (0, 16, 48, 256, 272):
        (xd, xgd, agd, god), keep = carve(step)
        assert [(t.data_ptr() - xd.data_ptr()) % 1024 for t in (xgd, agd, god)] == [step % 1024, 2 * step % 1024,
                                                                                    3 * step % 1024]
        h = capi.scan_fwd(xd, xgd, agd, lam_d)
        grads = capi.scan_bwd(xd, xgd, agd, lam_d, h, god)
        torch.cuda.synchronize()
        got = [h, *grads]
        if ref is None:
            ref = [t.clone() for t in got]
        else:
            for k, (a, b) in enumerate(zip(got, ref)):
                assert torch.equal(a, b), (step, k)
