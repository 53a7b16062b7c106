"""CPU-side checks: the C-ABI library loads and exports what the header declares, argument
validation answers without a GPU, and the Python host mirrors upstream's surface.  No
kernel is launched here."""

import ctypes
import math
import os
import re

import pytest
import torch

import hawk_pytorch_amd as hk
from hawk_pytorch_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "hawk_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(hawk_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = _lib.load()
    names = _declared_symbols()
    assert len(names) >= 12
    for name in names:
        assert hasattr(lib, name), name
        assert name in _lib.SIGNATURES, f"{name} declared in the header but not bound"
    assert sorted(_lib.SIGNATURES) == names
    assert lib.hawk_version() >= 100


def test_header_is_plain_c_and_links_against_the_library(tmp_path):
    """The boundary is a C ABI: the header must compile as C99 with no HIP or C++ headers, and a C
    program that only validates arguments (no GPU needed) must link and run against the .so."""
    import shutil
    import subprocess

    gcc = shutil.which("gcc")
    if gcc is None:
        pytest.skip("no gcc")
    src = tmp_path / "caller.c"
    src.write_text(
        '#include <stdio.h>\n#include <string.h>\n#include "hawk_hip.h"\n'
        "int main(void) {\n"
        "    char x[16];\n"
        "    if (hawk_version() < 100) return 1;\n"
        "    if (strcmp(hawk_status_string(HAWK_OK), \"ok\") != 0) return 2;\n"
        "    if (hawk_scan_workspace_bytes(8, 4096, 2560, HAWK_DTYPE_BF16) == 0) return 3;\n"
        "    if (hawk_rglru_scan_fwd(NULL, x, x, (const float*)x, x, 1, 1, 64, HAWK_DTYPE_BF16, NULL, 0, NULL)\n"
        "        != HAWK_ERR_NULL_POINTER) return 4;\n"
        "    if (hawk_gate_proj_supported(2560, 10) != 1 || hawk_gate_proj_supported(2560, 3) != 0) return 5;\n"
        '    puts("c caller ok");\n    return 0;\n}\n'
    )
    exe = tmp_path / "caller"
    libdir = os.path.dirname(_lib.LIB_PATH)
    _lib.load()  # builds the library if it is not there yet
    subprocess.run(
        [gcc, "-std=c99", "-Wall", "-Wextra", "-Werror", "-pedantic", "-I", os.path.join(ROOT, "include"), str(src),
         "-o", str(exe), "-L", libdir, "-l:" + os.path.basename(_lib.LIB_PATH), "-Wl,-rpath," + libdir,
         "-Wl,-rpath,/opt/rocm/lib", "-Wl,--allow-shlib-undefined"],
        check=True, capture_output=True, text=True)
    out = subprocess.run([str(exe)], check=True, capture_output=True, text=True)
    assert "c caller ok" in out.stdout


def test_status_strings_are_distinct():
    msgs = {_lib.status_string(s) for s in range(8)}
    assert len(msgs) == 8 and _lib.status_string(0) == "ok"
    assert "unknown" in _lib.status_string(99)


def test_argument_validation_needs_no_gpu():
    lib = _lib.load()
    buf = (ctypes.c_char * 4096)()
    p = (ctypes.addressof(buf) + 15) & ~15
    args = [p, p, p, p, p]
    assert lib.hawk_rglru_scan_fwd(None, p, p, p, p, 1, 8, 64, 0, None, 0, None) == _lib.HAWK_ERR_NULL_POINTER
    assert lib.hawk_rglru_scan_fwd(*args, 1, 8, 64, 7, None, 0, None) == _lib.HAWK_ERR_BAD_DTYPE
    assert lib.hawk_rglru_scan_fwd(*args, 0, 8, 64, 0, None, 0, None) == _lib.HAWK_ERR_BAD_SHAPE
    assert lib.hawk_rglru_scan_fwd(*args, 1, -3, 64, 0, None, 0, None) == _lib.HAWK_ERR_BAD_SHAPE
    assert lib.hawk_rglru_scan_fwd(p + 2, p, p, p, p, 1, 8, 64, 0, None, 0, None) == _lib.HAWK_ERR_ALIGNMENT
    # T spans several tiles but no workspace was given
    assert lib.hawk_rglru_scan_fwd(*args, 1, 4096, 64, 0, None, 0, None) == _lib.HAWK_ERR_WORKSPACE
    assert lib.hawk_rglru_scan_fwd(*args, 1, 4096, 64, 0, p, 256, None) == _lib.HAWK_ERR_WORKSPACE
    bwd = [p] * 10
    assert lib.hawk_rglru_scan_bwd(*bwd, 1, 8, 64, 0, None, 0, None) == _lib.HAWK_ERR_WORKSPACE
    assert lib.hawk_rglru_scan_bwd(*([None] + bwd[1:]), 1, 8, 64, 0, p, 1 << 20, None) == _lib.HAWK_ERR_NULL_POINTER
    assert lib.hawk_conv1d_fwd(p, p, p, None, p, 1, 8, 64, 9, 0, 0, None) == _lib.HAWK_ERR_BAD_SHAPE
    assert lib.hawk_conv1d_fwd(p, p, p, None, p, 1, 8, 64, 4, 0, 3, None) == _lib.HAWK_ERR_BAD_DTYPE
    assert lib.hawk_conv1d_bwd(p, p, p, p, p, p, 1, 8, 64, 4, 0, 0, None, 0, None) == _lib.HAWK_ERR_WORKSPACE
    assert lib.hawk_conv1d_step(None, p, p, p, p, 1, 64, 4, 0, 0, None) == _lib.HAWK_ERR_NULL_POINTER
    assert lib.hawk_rglru_step(p, p, p, p, p, p, 0, 64, 0, 0, None) == _lib.HAWK_ERR_BAD_SHAPE
    assert lib.hawk_scan_workspace_init(None, 1024, None) == _lib.HAWK_ERR_NULL_POINTER
    # mixed entry points: bf16 inputs with fp32 state is not an offered pair
    assert lib.hawk_rglru_scan_fwd_mixed(*args, 1, 8, 64, 0, 1, None, 0, None) == _lib.HAWK_ERR_BAD_DTYPE
    assert lib.hawk_rglru_scan_bwd_mixed(*bwd, 1, 8, 64, 0, 1, p, 1 << 20, None) == _lib.HAWK_ERR_BAD_DTYPE
    assert lib.hawk_rglru_scan_bwd_mixed(*bwd, 1, 8, 64, 1, 0, None, 0, None) == _lib.HAWK_ERR_WORKSPACE


def test_scan_shape_limits_are_checked_before_any_launch():
    """Row and tile byte offsets are formed in 32 bits inside the kernels: D and row strides
    beyond 2^24 elements are refused, as are shapes whose carries do not fit the fixed scratch
    array of the entry point that allocates nothing."""
    lib = _lib.load()
    buf = (ctypes.c_char * 4096)()
    p = (ctypes.addressof(buf) + 15) & ~15
    args = [p, p, p, p, p]
    big_d = (1 << 24) + 64
    assert lib.hawk_rglru_scan_fwd(*args, 1, 8, big_d, 0, None, 0, None) == _lib.HAWK_ERR_BAD_SHAPE
    assert lib.hawk_rglru_scan_fwd(*args, 1, 8, big_d, 1, None, 0, None) == _lib.HAWK_ERR_BAD_SHAPE
    assert lib.hawk_rglru_scan_bwd(*([p] * 10), 1, 8, big_d, 0, p, 1 << 20, None) == _lib.HAWK_ERR_BAD_SHAPE
    assert lib.hawk_scan_workspace_bytes(1, 8, big_d, 0) == 0
    assert lib.hawk_scan_workspace_bytes(1, 8, 1 << 24, 0) > 0
    assert lib.hawk_rglru_scan_fwd_static(*args, 1, 8, big_d, 0, None) == _lib.HAWK_ERR_BAD_SHAPE
    # 64 tiles in time x 8 x 2560 channels x 24 bytes = 31.5 MB of carry words > 16 MiB
    assert lib.hawk_rglru_scan_fwd_static(*args, 8, 8192, 2560, 0, None) == _lib.HAWK_ERR_SCRATCH_LIMIT
    assert lib.hawk_rglru_scan_fwd_static(None, p, p, p, p, 1, 8, 64, 0, None) == _lib.HAWK_ERR_NULL_POINTER
    # the size query states the limit exactly: the largest chain that fits, and one tile more
    limit = 16 << 20
    fits, over = 10922 * 128, 10923 * 128
    assert 0 < lib.hawk_rglru_scan_fwd_static_bytes(1, fits, 64, 0) <= limit
    assert lib.hawk_rglru_scan_fwd_static_bytes(1, over, 64, 0) > limit
    assert lib.hawk_rglru_scan_fwd_static_bytes(1, 128, 64, 0) == 0          # one tile: no carry words
    assert lib.hawk_rglru_scan_fwd_static_bytes(8, 4096, 2560, 0) <= 32 * 8 * 2560 * 24 + 1024
    assert lib.hawk_rglru_scan_fwd_static(*args, 1, over, 64, 0, None) == _lib.HAWK_ERR_SCRATCH_LIMIT
    if not torch.cuda.is_available():   # with a GPU this call would launch on the host buffer above
        assert lib.hawk_rglru_scan_fwd_static(*args, 1, fits, 64, 0, None) != _lib.HAWK_ERR_SCRATCH_LIMIT
    assert lib.hawk_rglru_scan_fwd_static(*args, 1, 8, 64, 5, None) == _lib.HAWK_ERR_BAD_DTYPE


def test_workspace_size_queries():
    lib = _lib.load()
    assert lib.hawk_scan_workspace_bytes(0, 1, 1, 0) == 0
    assert lib.hawk_scan_workspace_bytes(1, 1, 1, 5) == 0
    small = lib.hawk_scan_workspace_bytes(1, 64, 64, 0)
    big = lib.hawk_scan_workspace_bytes(8, 4096, 2560, 0)
    assert 256 <= small < big
    assert big % 256 == 0
    # a workspace sized for a shape serves every smaller shape
    assert lib.hawk_scan_workspace_bytes(4, 2048, 2560, 0) <= big
    assert lib.hawk_scan_workspace_bytes(8, 4096, 1280, 1) <= lib.hawk_scan_workspace_bytes(8, 4096, 2560, 1)
    assert lib.hawk_conv1d_bwd_workspace_bytes(8, 4096, 2560, 4) > 0
    assert lib.hawk_conv1d_bwd_workspace_bytes(8, 4096, 2560, 9) == 0


def test_no_cpu_fallback():
    x = torch.randn(1, 8, 64)
    lam = torch.randn(64)
    with pytest.raises((NotImplementedError, RuntimeError)):
        hk.fused_linear_scan(x, x, x, lam)
    with pytest.raises((NotImplementedError, RuntimeError)):
        hk.Conv1D(64, 4)(x)
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        hk.rglru_step(x[:, 0], x[:, 0], x[:, 0], lam, torch.zeros(1, 64))


def test_scan_wrapper_asserts_like_upstream():
    x = torch.randn(1, 8, 60)
    with pytest.raises(AssertionError, match="multiple of 64"):
        hk.sequential_scan_forward(x, x, x, torch.randn(60))
    y = torch.randn(1, 8, 64)
    with pytest.raises(AssertionError):
        hk.sequential_scan_forward(y, y[:, :4], y, torch.randn(64))


def test_rnn_cache_matches_upstream_layout_at_batch_one():
    c = hk.RNNCache(32, torch.device("cpu"), 4)
    assert c.recc_state.shape == (1, 1, 32) and c.conv_state.shape == (1, 3, 32)
    assert c.recc_state.dtype == torch.bfloat16 and c.conv_state.dtype == torch.bfloat16
    assert torch.isnan(c.recc_state.float()).all() and torch.isnan(c.conv_state.float()).all()
    assert c.current_cache_size == 0 and c.conv_cache_size == 3
    c.conv_state.zero_()
    rows = [torch.full((1, 1, 32), float(k + 1)) for k in range(4)]
    for r in rows:
        expect = torch.roll(c.conv_state, shifts=-1, dims=1)
        expect[:, -1, :] = r
        c.update_conv_cache(r)
        assert torch.equal(c.conv_state, expect)
    assert c.conv_state[0, :, 0].tolist() == [2.0, 3.0, 4.0]
    c.update_cache(rows[2])
    assert c.current_cache_size == 1 and float(c.recc_state[0, 0, 0]) == 3.0
    with pytest.raises(AssertionError):
        c.update_cache(torch.zeros(2, 1, 32))
    short = torch.arange(2 * 32, dtype=torch.float32).reshape(1, 2, 32)
    c.seed_conv_state(short)
    assert torch.equal(c.conv_state[:, 0].float(), torch.zeros(1, 32))
    assert torch.equal(c.conv_state[:, 1:].float(), short.bfloat16().float())
    assert "RNNCache" in repr(c)


def test_lambda_init_distribution():
    t = torch.empty(200000)
    hk.rnn_param_init(t, min_rad=0.9, max_rad=0.999)
    a2 = torch.exp(-2.0 * torch.nn.functional.softplus(t.double()))
    assert a2.min() >= 0.81 - 1e-6 and a2.max() <= 0.998001 + 1e-6
    assert abs(float(a2.mean()) - (0.81 + 0.998001) / 2) < 1e-3


def test_model_surface_and_parameter_count_of_the_readme_config():
    cfg = hk.HawkConfig(vocab_size=32000, hidden_size=512, intermediate_size=1024, recurrent_size=512,
                        num_hidden_layers=8, num_blocks=16, post_norm=False)
    assert cfg.conv_width == 4
    model = hk.HawkModel(cfg, use_cache=False)
    assert sum(p.numel() for p in model.parameters()) == 51_945_984
    sd = model.state_dict()
    expect = {
        "embed_tokens.weight": (32000, 512), "lm_head.weight": (32000, 512), "norm.weight": (512,),
        "layers.0.input_norm.weight": (512,), "layers.0.post_recurrent_norm.weight": (512,),
        "layers.0.recc.input_xy.weight": (1024, 512), "layers.0.recc.resid_proj.weight": (512, 512),
        "layers.0.recc.rg_lru_input_gate.w": (16, 32, 32), "layers.0.recc.rg_lru_input_gate.b": (16, 32),
        "layers.0.recc.rg_lru_a_gate.w": (16, 32, 32), "layers.0.recc.rg_lru_a_gate.b": (16, 32),
        "layers.0.recc.rg_lru_a_param": (512,), "layers.0.recc.conv1d.w": (4, 512),
        "layers.0.recc.conv1d.b": (512,), "layers.7.mlp.gate_up_proj.weight": (2048, 512),
        "layers.7.mlp.resid_proj.weight": (512, 1024),
    }
    for k, shape in expect.items():
        assert tuple(sd[k].shape) == shape, k
    assert len(sd) == 3 + 8 * 13
    assert sd["layers.3.recc.rg_lru_a_param"].dtype == torch.float32
    assert float(sd["lm_head.weight"].abs().max()) == 0.0
    assert float(sd["layers.0.recc.resid_proj.weight"].abs().max()) == 0.0
    with pytest.raises(NotImplementedError):
        hk.HawkConfig(10, 8, 8, 1, 8, 1, post_norm=True)
    assert len(model.new_cache(batch_size=3)) == 8


def test_custom_ops_have_shape_rules_for_tracing():
    from torch._subclasses.fake_tensor import FakeTensorMode

    with FakeTensorMode():
        x = torch.empty(2, 16, 64, dtype=torch.bfloat16, device="cuda")
        lam = torch.empty(64, device="cuda")
        h = torch.ops.hawk_amd.rglru_scan_fwd(x, x, x, lam, False)
        assert h.shape == x.shape and h.dtype == torch.bfloat16
        xf = torch.empty(2, 16, 64, device="cuda")
        hm = torch.ops.hawk_amd.rglru_scan_fwd(xf, xf, xf, lam, True)
        assert hm.dtype == torch.bfloat16
        gm = torch.ops.hawk_amd.rglru_scan_bwd(xf, xf, xf, lam, hm, hm)
        assert gm[0].dtype == torch.float32
        dx, dxg, dag, dlam = torch.ops.hawk_amd.rglru_scan_bwd(x, x, x, lam, h, h)
        assert dx.shape == x.shape and dlam.shape == (64,) and dlam.dtype == torch.float32
        w = torch.empty(4, 64, device="cuda")
        y = torch.ops.hawk_amd.conv1d_fwd(x, w, lam, None, True)
        assert y.dtype == torch.float32 and y.shape == x.shape
        gx, gw, gb = torch.ops.hawk_amd.conv1d_bwd(y, x, w)
        assert gx.dtype == torch.bfloat16 and gw.shape == (4, 64) and gb.shape == (64,)


def test_python_rule_for_fused_gate_projections_matches_the_library():
    from hawk_pytorch_amd import _lib
    from hawk_pytorch_amd.external import _GATE_BLOCK_WIDTHS

    lib = _lib.load()
    for D, nb in [(2560, 10), (512, 16), (512, 8), (512, 4), (512, 2), (512, 1), (96, 3), (100, 3), (4096, 16), (48, 3)]:
        python_rule = D % nb == 0 and (D // nb) in _GATE_BLOCK_WIDTHS
        assert bool(lib.hawk_gate_proj_supported(D, nb)) == python_rule, (D, nb)


def test_argument_validation_of_the_gated_and_projection_entry_points():
    lib = _lib.load()
    buf = (ctypes.c_char * 4096)()
    p = (ctypes.addressof(buf) + 15) & ~15
    E = _lib
    # gated scan forward: (x, xg, ag, lam, y, ldy, h, out, h_last, B, T, D, in, out, ws, bytes, stream)
    ok = [p, p, p, p, p, 64, p, p, None, 1, 8, 64, 0, 0, None, 0, None]

    def gf(**kw):
        a = list(ok)
        for k, v in kw.items():
            a[int(k[1:])] = v
        return lib.hawk_rglru_scan_gated_fwd(*a)

    assert gf(a4=None) == E.HAWK_ERR_NULL_POINTER            # y
    assert gf(a7=None) == E.HAWK_ERR_NULL_POINTER            # out
    assert gf(a5=63) == E.HAWK_ERR_BAD_SHAPE                 # row stride below D
    assert gf(a5=1 << 25) == E.HAWK_ERR_BAD_SHAPE            # row stride beyond the addressing limit
    assert gf(a12=1, a13=0, a10=4096) == E.HAWK_ERR_WORKSPACE  # (f32, bf16) is an offered pair: next check fails
    assert gf(a12=0, a13=1) == E.HAWK_ERR_BAD_DTYPE
    assert gf(a4=p + 1) == E.HAWK_ERR_ALIGNMENT              # y must be element aligned
    assert gf(a10=4096) == E.HAWK_ERR_WORKSPACE              # several tiles, no workspace
    # gated scan backward needs dy and a workspace
    gb = [p, p, p, p, p, 64, p, p, p, p, p, p, 64, p, 1, 8, 64, 0, 0, None, 0, None]
    assert lib.hawk_rglru_scan_gated_bwd(*gb) == E.HAWK_ERR_WORKSPACE
    gb[11] = None
    assert lib.hawk_rglru_scan_gated_bwd(*gb) == E.HAWK_ERR_NULL_POINTER
    # decode step with gate
    assert lib.hawk_rglru_step_gated(p, p, p, None, None, p, None, 64, p, None, p, 1, 64, 0, 0, None) \
        == E.HAWK_ERR_NULL_POINTER
    assert lib.hawk_rglru_step_gated(p, p, p, None, None, p, p, 32, p, None, p, 1, 64, 0, 0, None) \
        == E.HAWK_ERR_BAD_SHAPE
    # gate projections
    assert lib.hawk_gate_proj_fwd(p, p, None, p, None, p, p, 4, 1024, 2, 0, 1, 0, None) == E.HAWK_ERR_BAD_SHAPE
    assert lib.hawk_gate_proj_fwd(p, None, None, p, None, p, p, 4, 512, 4, 0, 1, 0, None) == E.HAWK_ERR_NULL_POINTER
    assert lib.hawk_gate_proj_fwd(p, p, None, p, None, p, p, 0, 512, 4, 0, 1, 0, None) == E.HAWK_ERR_BAD_SHAPE
    assert lib.hawk_gate_proj_fwd(p, p, None, p, None, p, p, 4, 512, 4, 0, 9, 0, None) == E.HAWK_ERR_BAD_DTYPE
    assert lib.hawk_gate_proj_bwd_input(p, p, p, p, None, p + 4, 4, 512, 4, 0, 1, 0, None) == E.HAWK_ERR_ALIGNMENT
    assert lib.hawk_gate_proj_bwd_weights(p, p, p, p, None, p, None, 4, 512, 4, 0, 0, None, 0, None) \
        == E.HAWK_ERR_WORKSPACE
    assert lib.hawk_gate_proj_bwd_weights(p, p, p, p, None, p, None, 4, 512, 4, 0, 0, p, 16, None) \
        == E.HAWK_ERR_WORKSPACE
    assert lib.hawk_gate_proj_bwd_weights_workspace_bytes(32768, 2560, 10) > 0
    assert lib.hawk_gate_proj_bwd_weights_workspace_bytes(32768, 2560, 7) == 0


def test_argument_validation_of_the_conv_front_and_the_strided_conv():
    lib = _lib.load()
    E = _lib
    p = 4096  # never dereferenced: every call below is refused before a launch
    ok = [p, 512, p, p, p, None, p, None, p, p, p, 2, 64, 256, 1, 4, 0, None]
    bad = list(ok); bad[12] = 31          # T < 32
    assert lib.hawk_conv_gate_proj_fwd(*bad) == E.HAWK_ERR_BAD_SHAPE
    bad = list(ok); bad[15] = 3           # temporal width other than 4
    assert lib.hawk_conv_gate_proj_fwd(*bad) == E.HAWK_ERR_BAD_SHAPE
    bad = list(ok); bad[1] = 255          # rows closer together than D
    assert lib.hawk_conv_gate_proj_fwd(*bad) == E.HAWK_ERR_BAD_SHAPE
    bad = list(ok); bad[1] = 260          # row stride not a multiple of 8
    assert lib.hawk_conv_gate_proj_fwd(*bad) == E.HAWK_ERR_BAD_SHAPE
    bad = list(ok); bad[14] = 3           # block width 256 / 3
    assert lib.hawk_conv_gate_proj_fwd(*bad) == E.HAWK_ERR_BAD_SHAPE
    bad = list(ok); bad[8] = None         # no conv output
    assert lib.hawk_conv_gate_proj_fwd(*bad) == E.HAWK_ERR_NULL_POINTER
    bad = list(ok); bad[0] = p + 2
    assert lib.hawk_conv_gate_proj_fwd(*bad) == E.HAWK_ERR_ALIGNMENT
    bad = list(ok); bad[16] = 5
    assert lib.hawk_conv_gate_proj_fwd(*bad) == E.HAWK_ERR_BAD_DTYPE
    # strided conv: strides below D or above 2^24 elements
    assert lib.hawk_conv1d_fwd_strided(p, 63, p, p, None, p, 64, 1, 8, 64, 4, 0, 0, None) == E.HAWK_ERR_BAD_SHAPE
    assert lib.hawk_conv1d_fwd_strided(p, 64, p, p, None, p, (1 << 24) + 1, 1, 8, 64, 4, 0, 0, None) \
        == E.HAWK_ERR_BAD_SHAPE
    assert lib.hawk_conv1d_bwd_strided(p, p, 64, p, p, 32, p, p, 1, 8, 64, 4, 0, 0, p, 1 << 20, None) \
        == E.HAWK_ERR_BAD_SHAPE
    assert lib.hawk_conv1d_bwd_strided(p, p, 64, p, p, 128, p, p, 1, 8, 64, 4, 0, 0, None, 0, None) \
        == E.HAWK_ERR_WORKSPACE


def test_argument_validation_of_the_block_core_entry_points():
    lib = _lib.load()
    E = _lib
    p = 4096  # never dereferenced: every call below is refused before a launch
    # xy, stride, conv_w, conv_b, w_i, b_i, w_a, b_a, w_dtype, w_bf16, a_param, u, xg, ag, h, out, h_last,
    # B, T, D, nb, W, scan_ws, bytes, stream
    ok = [p, 512, p, p, p, None, p, None, 1, p, p, p, p, p, None, p, None, 2, 64, 256, 1, 4, p, 1 << 20, None]
    for idx, what in ((18, 31), (21, 3), (1, 511), (1, 516), (20, 3), (19, 252)):   # T, width, stride, stride % 8, blocks, D % 8
        bad = list(ok); bad[idx] = what
        assert lib.hawk_block_core_fwd(*bad) == E.HAWK_ERR_BAD_SHAPE, (idx, what)
    for idx in (0, 2, 3, 4, 6, 10, 11, 12, 13, 15):
        bad = list(ok); bad[idx] = None
        assert lib.hawk_block_core_fwd(*bad) == E.HAWK_ERR_NULL_POINTER, idx
    bad = list(ok); bad[8] = 7
    assert lib.hawk_block_core_fwd(*bad) == E.HAWK_ERR_BAD_DTYPE
    bad = list(ok); bad[15] = p + 8
    assert lib.hawk_block_core_fwd(*bad) == E.HAWK_ERR_ALIGNMENT
    # xy, stride, u, xg, ag, h, conv_w, w_i, w_a, w_dtype, a_param, grad_out, d_xy, stride, du, dxg, dag, dcw, dcb,
    # dw_i, db_i, dw_a, db_a, da_param, B, T, D, nb, W, 3 x (workspace, bytes), stream
    ok = [p, 512, p, p, p, p, p, p, p, 0, p, p, p, 512, p, p, p, p, p, p, None, p, None, p, 2, 64, 256, 1, 4,
          p, 1 << 20, p, 1 << 20, p, 1 << 20, None]
    for idx, what in ((28, 9), (28, 0), (1, 511), (13, 511), (13, 516), (27, 3), (26, 252), (24, 70000)):
        bad = list(ok); bad[idx] = what
        assert lib.hawk_block_core_bwd(*bad) == E.HAWK_ERR_BAD_SHAPE, (idx, what)
    for idx in (0, 2, 3, 4, 5, 6, 7, 8, 10, 11, 12, 14, 15, 16, 17, 18, 19, 21, 23):
        bad = list(ok); bad[idx] = None
        assert lib.hawk_block_core_bwd(*bad) == E.HAWK_ERR_NULL_POINTER, idx
    for idx in (29, 31, 33):
        bad = list(ok); bad[idx] = None
        assert lib.hawk_block_core_bwd(*bad) == E.HAWK_ERR_WORKSPACE, idx
    bad = list(ok); bad[9] = 7
    assert lib.hawk_block_core_bwd(*bad) == E.HAWK_ERR_BAD_DTYPE
    bad = list(ok); bad[12] = p + 4
    assert lib.hawk_block_core_bwd(*bad) == E.HAWK_ERR_ALIGNMENT
    # both gates' weights in one launch
    assert lib.hawk_gate_weights_to_bf16(p, p, p, None, 2, 64, None) == E.HAWK_ERR_NULL_POINTER
    assert lib.hawk_gate_weights_to_bf16(p, p, p, p, 2, 6, None) == E.HAWK_ERR_BAD_SHAPE
    assert lib.hawk_gate_weights_to_bf16(p, p, p + 2, p, 2, 64, None) == E.HAWK_ERR_ALIGNMENT


def test_argument_validation_of_the_fused_decode_step():
    lib = _lib.load()
    buf = (ctypes.c_char * 4096)()
    p = (ctypes.addressof(buf) + 15) & ~15
    E = _lib
    # (conv_state, x_new, ldx, conv_w, conv_b, w_i, b_i, w_a, b_a, a_param, y, ldy, recc_state, out,
    #  B, D, num_blocks, W, dtype, w_dtype, state_dtype, stream)
    ok = [p, p, 512, p, p, p, None, p, None, p, p, 512, p, p, 1, 256, 2, 4, 0, 0, 0, None]

    def step(**kw):
        a = list(ok)
        for k, v in kw.items():
            a[int(k[1:])] = v
        return lib.hawk_decode_core_step(*a)

    assert step(a1=None) == E.HAWK_ERR_NULL_POINTER          # x_new
    assert step(a0=None) == E.HAWK_ERR_NULL_POINTER          # a window of 3 rows needs its state
    assert step(a0=None, a17=1, a1=p + 2) == E.HAWK_ERR_ALIGNMENT  # no window, no state: the next check fails
    assert step(a18=1) == E.HAWK_ERR_BAD_DTYPE               # activations must be bf16
    assert step(a19=7) == E.HAWK_ERR_BAD_DTYPE
    assert step(a17=9) == E.HAWK_ERR_BAD_SHAPE               # window too wide
    assert step(a16=3) == E.HAWK_ERR_BAD_SHAPE               # 256 channels do not split in 3 blocks
    assert step(a2=255) == E.HAWK_ERR_BAD_SHAPE              # row stride below D
    assert step(a2=260) == E.HAWK_ERR_BAD_SHAPE              # rows of x_new must stay 16-byte aligned
    assert step(a11=100) == E.HAWK_ERR_BAD_SHAPE
    assert step(a1=p + 2) == E.HAWK_ERR_ALIGNMENT
    assert step(a10=p + 1) == E.HAWK_ERR_ALIGNMENT           # y must be element aligned
    assert lib.hawk_decode_core_supported(2560, 10, 4) == 1
    assert lib.hawk_decode_core_supported(2560, 10, 9) == 0
    assert lib.hawk_decode_core_supported(2560, 7, 4) == 0


def test_bench_refuses_more_than_one_gpu():
    import subprocess
    import sys

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"],
                       capture_output=True, text=True, timeout=300, cwd=root)
    assert r.returncode == 2
    assert "one GPU" in r.stderr and r.stdout.strip() == ""


def test_activation_placement_steps_through_the_kilobyte(monkeypatch):
    """_lib.activation_empty: large tensors start 256 bytes further on (modulo 1 KiB) from one call
    to the next, are contiguous and 16-byte aligned; small ones and HAWK_STAGGER_BYTES=0 give a
    plain torch.empty."""
    from hawk_pytorch_amd import _lib

    monkeypatch.delenv("HAWK_STAGGER_BYTES", raising=False)
    shape = (4, 2048, 1024)
    ts = [_lib.activation_empty(shape, torch.bfloat16, "cpu") for _ in range(6)]
    pos = [t.data_ptr() % 1024 for t in ts]
    assert all((b - a) % 1024 == 256 for a, b in zip(pos, pos[1:])), pos
    for t in ts:
        assert t.shape == shape and t.is_contiguous() and t.data_ptr() % 16 == 0 and t.dtype == torch.bfloat16
        t.zero_()   # the whole view lies inside its buffer
    f = _lib.activation_empty((2048, 2048), torch.float32, "cpu")
    assert (f.data_ptr() - ts[-1].data_ptr()) % 1024 == 256 and f.is_contiguous()
    small = _lib.activation_empty((8, 64), torch.bfloat16, "cpu")
    assert small.storage_offset() == 0 and small.numel() == 512
    empty = _lib.activation_empty((0,), torch.bfloat16, "cpu")
    assert empty.numel() == 0
    monkeypatch.setenv("HAWK_STAGGER_BYTES", "0")
    assert _lib.activation_empty(shape, torch.bfloat16, "cpu").storage_offset() == 0
    monkeypatch.setenv("HAWK_STAGGER_BYTES", "100")
    with pytest.raises(ValueError):
        _lib.activation_empty(shape, torch.bfloat16, "cpu")
    assert _lib.activation_empty((8, 64), torch.bfloat16, "cpu").numel() == 512   # small: the setting is not read
