"""CPU-side tests of the drop-in boundary: the C-ABI library loads, exports every symbol the header
declares, validates arguments on the host (no GPU touched), and its index-map hooks are bit-exact
against the oracle.  The module layer keeps the reference's state_dict layout."""
import ctypes
import os
import re

import numpy as np
import pytest
import torch
from hypothesis import given, settings, strategies as st

import oracle

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol(pkg):
    header = open(os.path.join(ROOT, "include", "aeris_hip.h")).read()
    declared = set(re.findall(r"\b(aeris_[a-z0-9_]+)\s*\(", header))
    assert declared, "header declares nothing?"
    lib = pkg._lib.lib()
    for name in declared:
        assert hasattr(lib, name), f"{name} declared in include/aeris_hip.h but not exported"
    assert declared == set(pkg._lib.SIGNATURES), "ctypes signature table and header disagree"
    assert lib.aeris_version() >= 1


CASES = [(1, 4, 8, 2, 4, 0, 0), (1, 4, 8, 2, 4, 1, 2), (2, 6, 6, 3, 2, 1, 1), (1, 32, 64, 8, 8, 4, 4),
         (1, 180, 360, 12, 12, 6, 6), (2, 64, 96, 16, 16, 8, 8)]


@pytest.mark.parametrize("case", CASES)
def test_window_index_map_bit_exact(pkg, case):
    np.testing.assert_array_equal(pkg.ops.window_index_map(*case), oracle.window_token_index(*case))


def test_window_index_map_full_grid(pkg):
    got = pkg.ops.window_index_map(1, 720, 1440, 16, 16, 8, 8)
    np.testing.assert_array_equal(got, oracle.window_token_index(1, 720, 1440, 16, 16, 8, 8))
    assert got.shape == (4050, 256)


@settings(max_examples=30, deadline=None)
@given(B=st.integers(1, 2), ny=st.integers(1, 4), nx=st.integers(1, 4), wy=st.integers(1, 6), wx=st.integers(1, 6), data=st.data())
def test_window_index_map_hypothesis(pkg, B, ny, nx, wy, wx, data):
    sy, sx = data.draw(st.integers(0, wy - 1)), data.draw(st.integers(0, wx - 1))
    case = (B, ny * wy, nx * wx, wy, wx, sy, sx)
    np.testing.assert_array_equal(pkg.ops.window_index_map(*case), oracle.window_token_index(*case))


@pytest.mark.parametrize("ws", [(2, 2), (3, 5), (8, 8), (12, 12), (16, 16)])
def test_relative_position_index_bit_exact(pkg, ws):
    np.testing.assert_array_equal(pkg.ops.relative_position_index(*ws), oracle.relative_position_index(*ws))


@pytest.mark.parametrize("geo", [(8, 12, 4, 4, 2, 2), (32, 64, 8, 8, 4, 4), (180, 360, 12, 12, 6, 6), (16, 16, 8, 8, 4, 0)])
def test_shift_regions_reproduce_the_oracle_mask(pkg, geo):
    H, W, wy, wx, sy, sx = geo
    ids = pkg.ops.shift_region_ids(*geo)  # [nW, L]
    mask = np.where(ids[:, :, None] != ids[:, None, :], np.float32(-100.0), np.float32(0.0))
    np.testing.assert_array_equal(mask, oracle.shift_attention_mask(*geo))


def test_argument_validation_needs_no_gpu(pkg):
    L = pkg._lib
    lib = L.lib()
    buf = (ctypes.c_char * 4096)()
    p = ctypes.addressof(buf)
    p16 = (p + 15) // 16 * 16
    # index maps
    assert lib.aeris_window_index_map(1, 10, 8, 4, 4, 0, 0, p) == L.EINVAL  # 10 % 4 != 0
    assert "multiple" in L.last_error()
    assert lib.aeris_window_index_map(1, 8, 8, 4, 4, 4, 0, p) == L.EINVAL  # shift >= window
    assert lib.aeris_window_index_map(1, 8, 8, 4, 4, 0, 0, None) == L.EINVAL
    assert lib.aeris_relative_position_index(0, 4, p) == L.EINVAL
    # attention
    f = lib.aeris_window_attention_fwd
    assert f(None, p16, None, 1, 16, 16, 2, 64, 16, 16, 0, 0, 0, 0.125, None) == L.EINVAL
    assert f(p16 + 2, p16, None, 1, 16, 16, 2, 64, 16, 16, 0, 0, 0, 0.125, None) == L.EINVAL  # misaligned
    # the reference's 60x60 x 128 runs on the streaming kernel, but not with a bias table or the shift mask
    assert f(p16, p16, p16, 1, 60, 60, 12, 128, 60, 60, 0, 0, 0, 0.1, None) == L.EUNSUPPORTED
    assert "no kernel" in L.last_error() and "bias" in L.last_error()
    assert f(p16, p16, None, 1, 60, 60, 12, 128, 60, 60, 30, 30, 1, 0.1, None) == L.EUNSUPPORTED
    assert f(p16, p16, None, 1, 65, 65, 2, 64, 65, 65, 0, 0, 0, 0.1, None) == L.EUNSUPPORTED  # 4225 tokens per window
    assert f(p16, p16, None, 1, 16, 16, 2, 96, 16, 16, 0, 0, 0, 0.1, None) == L.EUNSUPPORTED  # head_dim 96
    assert f(p16, p16, None, 1, 16, 16, 2, 64, 16, 16, 0, 0, 0, 0.0, None) == L.EINVAL  # scale
    assert f(p16, p16, None, 1, 16, 20, 2, 64, 16, 16, 0, 0, 0, 0.125, None) == L.EINVAL  # grid not a multiple
    # norm
    g = lib.aeris_norm_modulate_fwd
    assert g(p16, 0, p16, 0, None, None, 0, None, None, 0, 1, 4, 64, 0, 0, 1e-5, None) == L.EINVAL  # gamma NULL
    assert g(p16, 0, p16, 0, p16, None, 0, None, None, 0, 1, 4, 60, 0, 0, 1e-5, None) == L.EUNSUPPORTED  # d % 8
    assert g(p16, 7, p16, 0, p16, None, 0, None, None, 0, 1, 4, 64, 0, 0, 1e-5, None) == L.EINVAL  # dtype
    assert g(p16, 0, p16, 0, p16, None, 0, None, None, 0, 1, 4, 64, 5, 0, 1e-5, None) == L.EINVAL  # kind
    assert g(p16, 0, p16, 0, p16 + 2, None, 0, None, None, 0, 1, 4, 64, 0, 0, 1e-5, None) == L.EINVAL  # gamma not 16-byte aligned
    assert g(p16, 0, p16, 0, p16, None, 0, p16 + 4, None, 64, 1, 4, 64, 0, 0, 1e-5, None) == L.EINVAL  # shift not aligned
    assert g(p16, 0, p16, 0, p16, None, 0, p16, p16, 66, 1, 4, 64, 0, 0, 1e-5, None) == L.EINVAL  # mod_batch_stride % 4
    # gemm
    h = lib.aeris_gemm_fwd
    assert h(p16, p16, p16, None, None, None, 8, 8, 100, 8, 0, 0, 0, 0, 0, None) == L.EUNSUPPORTED  # K % 64
    assert h(p16, p16, p16, None, None, None, 8, 8, 64, 4, 0, 0, 0, 0, 0, None) == L.EINVAL  # ldc < N
    assert h(p16, p16, p16, None, None, None, 0, 8, 64, 8, 0, 0, 0, 0, 0, None) == L.EINVAL  # M
    assert h(p16, p16, p16, None, None, None, 8, 8, 64, 8, 9, 0, 0, 0, 0, None) == L.EINVAL  # act
    # head-plane variants: same checks, plus the plane geometry
    fh = lib.aeris_window_attention_heads_fwd
    assert fh(None, p16, None, 1, 16, 16, 2, 64, 16, 16, 0, 0, 0, 0.125, 0, 256 * 64, None) == L.EINVAL
    assert fh(p16, p16, None, 1, 16, 16, 2, 64, 16, 16, 0, 0, 0, 0.125, 1, 256 * 64 - 8, None) == L.EINVAL  # planes overlap
    assert "plane_stride" in L.last_error()
    assert fh(p16, p16, None, 1, 16, 16, 2, 64, 16, 16, 0, 0, 0, 0.125, 0, 256 * 64 + 4, None) == L.EINVAL  # not 16-byte planes
    assert fh(p16, p16, None, 1, 16, 16, 2, 96, 16, 16, 0, 0, 0, 0.1, 0, 256 * 96, None) == L.EUNSUPPORTED  # head_dim 96
    hh = lib.aeris_gemm_heads_fwd
    assert hh(p16, p16, p16, None, 8, 128, 100, 64, 8 * 64, 1.0, 0, None) == L.EUNSUPPORTED  # K % 64
    assert hh(p16, p16, p16, None, 8, 100, 64, 64, 8 * 64, 1.0, 0, None) == L.EINVAL  # N % head_dim
    assert hh(p16, p16, p16, None, 8, 128, 64, 60, 8 * 60, 1.0, 0, None) == L.EINVAL  # head_dim % 8
    assert hh(p16, p16, p16, None, 8, 128, 64, 64, 8 * 64 - 8, 1.0, 0, None) == L.EINVAL  # planes overlap
    assert hh(p16, None, p16, None, 8, 128, 64, 64, 8 * 64, 1.0, 0, None) == L.EINVAL  # W NULL
    assert hh(p16, p16, p16, None, 8, 128, 64, 64, 8 * 64, 0.18, 3, None) == L.EINVAL  # more query planes than planes
    assert "q_planes" in L.last_error()
    assert hh(p16, p16, p16, None, 8, 128, 64, 64, 8 * 64, 0.0, 1, None) == L.EINVAL  # q_scale must be positive
    assert hh(p16, p16, p16, None, 8, 128, 64, 64, 8 * 64, float("nan"), 1, None) == L.EINVAL
    # fused to_qkv + window attention
    qa, qb, qp = lib.aeris_qkv_window_attention_fwd, lib.aeris_qkv_attention_bias_bytes, lib.aeris_qkv_attention_prepare_bias
    assert qb(24, 16, 16) == 24 * 961 * 16 and qb(24, 12, 12) == 0 and qb(0, 16, 16) == 0
    assert qp(None, 24, 16, 16, p16, None) == L.EINVAL and qp(p16, 24, 8, 8, p16, None) == L.EUNSUPPORTED
    okq = (p16, p16, None, None, p16, 1, 32, 32, 2, 64, 256, 16, 16, 8, 8, 1, 0.125, None)
    def withq(i, v):
        a = list(okq); a[i] = v; return a
    assert qa(*withq(0, None)) == L.EINVAL and qa(*withq(4, None)) == L.EINVAL  # y / out NULL
    assert qa(*withq(2, p16 + 2)) == L.EINVAL  # projection bias not 8-byte aligned
    assert qa(*withq(9, 128)) == L.EUNSUPPORTED and qa(*withq(10, 320)) == L.EUNSUPPORTED  # head_dim, K % 128
    assert qa(*withq(10, 128)) == L.EUNSUPPORTED  # fewer than four k-tiles
    assert qa(*withq(11, 32)) == L.EUNSUPPORTED  # 32x16 windows
    assert "aeris_gemm_heads_fwd" in L.last_error()  # the message names the two-kernel path to use instead
    assert qa(*withq(13, 16)) == L.EINVAL  # shift outside the window
    assert qa(*withq(16, 0.0)) == L.EINVAL  # scale
    # fused output stage
    osf, osw = lib.aeris_output_stage_fwd, lib.aeris_output_stage_workspace_bytes
    assert osw(69, 1536, 1) == 1536 * 80 * 4 + 80 * 8 and osw(69, 1536, 4) == 4 * osw(69, 1536, 1)
    assert osw(81, 1536, 1) == 0 and osw(69, 1500, 1) == 0 and osw(69, 1536, 0) == 0  # unsupported shapes: no size
    ok = (p16, L.F32, p16, None, L.F32, None, None, 0, p16, p16, 1, 128, 69, 1536, L.NORM_RMS, 1e-6, p16, osw(69, 1536, 1), None)
    def with_(i, v):
        a = list(ok); a[i] = v; return a
    assert osf(*with_(0, None)) == L.EINVAL and osf(*with_(8, None)) == L.EINVAL  # x / head_w NULL
    assert osf(*with_(12, 81)) == L.EUNSUPPORTED and osf(*with_(13, 1500)) == L.EUNSUPPORTED
    assert osf(*with_(17, osw(69, 1536, 1) - 1)) == L.EINVAL and "workspace" in L.last_error()
    assert osf(*with_(16, None)) == L.EINVAL
    assert osf(*with_(14, 7)) == L.EINVAL  # norm kind
    # one modulation row per batch entry: rows_per_batch must be a multiple of the 64-row tile
    a = list(ok); a[5] = p16; a[7] = 1536; a[10] = 2; a[11] = 100; a[17] = osw(69, 1536, 2)
    assert osf(*a) == L.EUNSUPPORTED
    # small ops
    assert lib.aeris_modulation_linear_fwd(p16, p16, None, p16, 1, 8, 12, 0, 0, None) == L.EUNSUPPORTED
    assert lib.aeris_timestep_embedding_fwd(p16, p16, 1, 7, 10000.0, None) == L.EINVAL
    assert lib.aeris_embed_prepare_fwd(p16, None, p16, 4, 0, 138, 128, 0, None) == L.EINVAL  # K_pad < C
    assert lib.aeris_embed_prepare_fwd(p16, None, p16, 4, 0, 138, 384, 1, None) == L.EINVAL  # split: K_pad < 3 C + 2
    assert lib.aeris_embed_concat_fwd(p16, 69, 1.0, p16, 69, None, p16, 4, 0, 128, 0, None) == L.EINVAL  # K_pad < C0 + C1
    assert lib.aeris_embed_concat_fwd(p16, 69, 1.0, p16, 69, None, p16, 4, 0, 384, 1, None) == L.EINVAL  # split: too narrow
    assert lib.aeris_embed_concat_fwd(p16, 69, 0.0, p16, 69, None, p16, 4, 0, 192, 0, None) == L.EINVAL  # div0 == 0
    assert lib.aeris_embed_concat_fwd(p16, 69, 1.0, None, 69, None, p16, 4, 0, 192, 0, None) == L.EINVAL  # x1 NULL
    # fused input stage
    isw, isp, isf = lib.aeris_input_stage_weight_bytes, lib.aeris_input_stage_pack_weight, lib.aeris_input_stage_fwd
    assert isw(138, 1536) == 96 * 5 * 2048 and isw(31, 64) == 4 * 1 * 2048 and isw(32, 64) == 4 * 2 * 2048
    assert isw(160, 1536) == 0 and isw(138, 1500) == 0 and isw(0, 64) == 0  # unsupported shapes: no size
    assert isp(None, None, p16, 138, 1536, None) == L.EINVAL and isp(p16, None, p16, 160, 1536, None) == L.EUNSUPPORTED
    ok = (p16, 69, 1.0, p16, 69, None, 0, p16, p16, L.F32, 256, 1536, None)
    assert isf(*with_of(ok, 0, None)) == L.EINVAL and isf(*with_of(ok, 7, None)) == L.EINVAL  # x0 / packed NULL
    assert isf(*with_of(ok, 3, None)) == L.EINVAL  # C1 > 0 without x1
    assert isf(*with_of(ok, 2, 0.0)) == L.EINVAL  # div0 == 0
    assert isf(*with_of(ok, 1, 100)) == L.EUNSUPPORTED and isf(*with_of(ok, 11, 1500)) == L.EUNSUPPORTED
    assert isf(*with_of(ok, 10, 0)) == L.EINVAL and isf(*with_of(ok, 9, 7)) == L.EINVAL  # M, out dtype
    a = list(ok); a[5] = p16; a[6] = 0
    assert isf(*a) == L.EINVAL  # ape without rows
    a[6] = 32
    assert isf(*a) == L.EUNSUPPORTED and "positional" in L.last_error()
    with pytest.raises(pkg.AerisError):
        L.call("aeris_window_index_map", 1, 10, 8, 4, 4, 0, 0, p)


def with_of(args, i, v):
    a = list(args)
    a[i] = v
    return a


def test_ops_refuse_cpu_tensors(pkg):
    x = torch.zeros(1, 4, 64, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="GPU"):
        pkg.ops.norm_modulate(x, torch.ones(64, dtype=torch.bfloat16))
    with pytest.raises(RuntimeError, match="GPU"):
        pkg.ops.gemm(x, torch.zeros(64, 64, dtype=torch.bfloat16))


def test_ref_state_dict_layout_matches_reference(pkg):
    """Key names, shapes and dtypes as listed for LocalAERIS (model.py:342,170,387-392,410-418,452-466)."""
    d, heads, hd, Hd, cin, cout = 64, 2, 32, 128, 10, 5
    m = pkg.LocalAERIS(device_mesh=None, heads=heads, dim=d, head_dim=hd, mlp_dim=Hd, window_size=(8, 8),
                       image_shape=(16, 16), rope_base=10_000, sublayers=2, sinusoidal_emb_max_period=10_000,
                       n_layers=4, model_in_channels=cin, model_out_channels=cout)
    sd = m.state_dict()
    inner = heads * hd
    want = {"input_stage.proj.weight": ((d, cin), torch.float32), "input_stage.proj.bias": ((d,), torch.float32),
            "input_stage.ape.inv_freq": ((3,), torch.float32),
            "output_stage.norm.weight": ((d,), torch.float32),
            "output_stage.modulation.0.weight": ((d, d), torch.float32), "output_stage.modulation.0.bias": ((d,), torch.float32),
            "output_stage.modulation.2.weight": ((2 * d, d), torch.float32), "output_stage.modulation.2.bias": ((2 * d,), torch.float32),
            "output_stage.head.weight": ((cout, d), torch.float32)}
    for i in range(2):
        for j in range(2):
            p = f"layers.{i}.modulelist.{j}."
            want.update({p + "0.weight": ((d,), torch.bfloat16), p + "1.to_qkv.weight": ((3 * inner, d), torch.bfloat16),
                         p + "1.wo.weight": ((d, inner), torch.bfloat16), p + "2.weight": ((d,), torch.bfloat16),
                         p + "3.w1.weight": ((2 * Hd, d), torch.bfloat16), p + "3.w2.weight": ((d, Hd), torch.bfloat16),
                         # the modulation MLP keeps f32 parameters (same keys and shapes; a bf16 checkpoint loads without loss)
                         p + "4.modulation.0.weight": ((d, d), torch.float32), p + "4.modulation.0.bias": ((d,), torch.float32),
                         p + "4.modulation.2.weight": ((6 * d, d), torch.float32), p + "4.modulation.2.bias": ((6 * d,), torch.float32)})
    assert set(sd.keys()) == set(want.keys())
    for k, (shape, dt) in want.items():
        assert tuple(sd[k].shape) == shape and sd[k].dtype == dt, k


def test_spec_state_dict_layout(pkg):
    layer = pkg.SwinLayer(None, 64, 2, 32, 256, (8, 8), (16, 16), True, 10_000, preset="spec", mod_ways=2)
    keys = set(layer.state_dict().keys())
    p = "modulelist.0."
    assert keys == {p + k for k in ("0.weight", "0.bias", "1.to_qkv.weight", "1.to_qkv.bias", "1.wo.weight", "1.wo.bias",
                                    "1.relative_position_bias_table", "2.weight", "2.bias", "3.fc1.weight", "3.fc1.bias",
                                    "3.fc2.weight", "3.fc2.bias", "4.modulation.0.weight", "4.modulation.0.bias",
                                    "4.modulation.2.weight", "4.modulation.2.bias")}
    assert layer.state_dict()[p + "1.relative_position_bias_table"].shape == (225, 2)
    assert layer.state_dict()[p + "4.modulation.2.weight"].shape == (4 * 64, 64)
    assert layer.default_shift() == (4, 4)


def test_convert_inference_checkpoint_roundtrip(pkg, tmp_path):
    kw = dict(device_mesh=None, heads=2, dim=64, head_dim=32, mlp_dim=128, window_size=(8, 8), image_shape=(16, 16),
              rope_base=10_000, sublayers=1, sinusoidal_emb_max_period=10_000, n_layers=4, model_in_channels=10,
              model_out_channels=5)
    src = pkg.LocalAERIS(**kw)
    N = 4
    stages = [dict() for _ in range(N)]
    for k, v in src.state_dict().items():
        if k.startswith("input_stage."):
            stages[0][k[len("input_stage."):]] = v
        elif k.startswith("output_stage."):
            stages[N - 1][k[len("output_stage."):]] = v
        else:
            _, i, rest = k.split(".", 2)
            stages[int(i) + 1][rest] = v
    stages[0]["latent_embed.weight"] = torch.zeros(3)  # stray entries the converter must drop (model.py:483,488)
    stages[1]["modulelist.0.1.norm.weight"] = torch.zeros(3)
    for k, s in enumerate(stages):
        torch.save({"ema_state_dict": s}, tmp_path / f"checkpoint_PP{k}.pth")
    dst = pkg.LocalAERIS(**kw)
    pkg.convert_inference_checkpoint(str(tmp_path), N, dst)
    for k, v in src.state_dict().items():
        assert torch.equal(dst.state_dict()[k], v), k
    del stages[2]["modulelist.0.3.w2.weight"]
    torch.save({"ema_state_dict": stages[2]}, tmp_path / "checkpoint_PP2.pth")
    with pytest.raises(KeyError):
        pkg.convert_inference_checkpoint(str(tmp_path), N, dst)


def test_host_sigma_schedule_matches_oracle(pkg):
    torch.testing.assert_close(pkg.sigma_schedule(10), oracle.sigma_schedule(10), rtol=0, atol=0)


def test_bench_refuses_more_than_one_gpu():
    """The whole grid runs on one GPU; bench.py says so instead of pretending to scale."""
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=300)
    assert r.returncode == 2
    assert "ONE GPU" in (r.stdout + r.stderr)


def test_rollout_refuses_steps_beyond_the_forecast(pkg):
    """The forecast-step counter lives on the device; the host-side mirror keeps run() from indexing forcings,
    latents or the state store past their end."""
    import importlib
    sm = importlib.import_module(pkg.__name__ + ".sampler")
    ro = sm._Rollout(torch.zeros(1, 4, 3), 2, None, None, None, None, None, None, None, None)
    calls = []
    ro.step = lambda: calls.append(1)
    ro.run(1)
    ro.run()
    assert len(calls) == 2
    with pytest.raises(ValueError, match="forecast steps are done"):
        ro.run(1)
    ro.reset()
    ro.run(2)
    assert len(calls) == 4
    with pytest.raises(ValueError):
        sm._Rollout(torch.zeros(1, 4, 3), 2, None, None, None, None, torch.zeros(2, 1, 4, 1), None, None, None)  # forcing too short
