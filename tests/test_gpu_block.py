"""GPU parity of the Swin block, the full denoiser and the sampler against the fp32 CPU oracle.

Bar (from the benchmark definition): bf16 output within relative L2 <= 1e-2 of the fp32 oracle on identical
seeded inputs; the attention-branch and MLP-branch outputs are compared as well because with the plain
random init (std 0.02) the residual dominates the block output.
"""
import math

import pytest
import torch

import oracle
from oracle import OracleConfig
from helpers import branch_tap, make_layer, make_model, rel_l2, max_abs

pytestmark = pytest.mark.gpu

CONFIG0 = dict(dim=128, heads=4, head_dim=32, mlp_dim=512, window_size=(8, 8), image_shape=(32, 64))
CONFIG1 = dict(dim=512, heads=8, head_dim=64, mlp_dim=2048, window_size=(12, 12), image_shape=(180, 360))
SMALL16 = dict(dim=256, heads=4, head_dim=64, mlp_dim=1024, window_size=(16, 16), image_shape=(32, 48))
MAX_ABS_OVER_RMS = 0.1  # bound on the largest element-wise deviation, in units of the oracle tensor's rms


def _run_block(pkg, cuda, cfg, seed, nontrivial, shifted, x_dtype=torch.bfloat16, B=1):
    sd = oracle.init_block_weights(cfg, seed, nontrivial=nontrivial)
    g = torch.Generator().manual_seed(seed + 100)
    S = cfg.image_shape[0] * cfg.image_shape[1]
    x = torch.randn(B, S, cfg.dim, generator=g)
    t = torch.randn(1, cfg.dim, generator=g) if cfg.mod_ways else None
    shift = (cfg.window_size[0] // 2, cfg.window_size[1] // 2) if shifted else (0, 0)
    xin = x.to(x_dtype)
    ref, ref_a, ref_m = oracle.block_forward(cfg, sd, xin.float(), t, shift, return_branches=True)
    layer = make_layer(pkg, cfg, sd, cuda, shifted)
    br = {}
    out = layer(xin.to(cuda), None if t is None else t.to(cuda), tap=branch_tap(pkg, br))
    torch.cuda.synchronize()
    assert out.dtype == x_dtype and out.shape == x.shape
    # the largest single deviation, in units of the compared tensor's rms: a bf16 result rounds by up to 2^-9 of its
    # value, about 0.01 rms on the largest elements of a normal tensor; an element off by a tenth of an rms is a defect
    # that a relative L2 over a million elements would not show
    for name, got, want in (("block", out, ref), ("attention branch", br["attn"].view_as(ref_a), ref_a),
                            ("MLP branch", br["mlp"].view_as(ref_m), ref_m)):
        worst = max_abs(got, want) / float(want.double().pow(2).mean().sqrt())
        print(f"{name}: rel-L2 {rel_l2(got, want):.3e}, max-abs / rms {worst:.3e}")
        assert worst <= MAX_ABS_OVER_RMS, (name, worst)
    return rel_l2(out, ref), rel_l2(br["attn"].view_as(ref_a), ref_a), rel_l2(br["mlp"].view_as(ref_m), ref_m)


@pytest.mark.parametrize("shifted", [False, True])
def test_config0_block(pkg, cuda, shifted):
    """configs[0]: 32x64 grid, dim 128, 4x32 heads, 8x8 windows, shift 4, rel-pos bias, mask, LN, GELU x4."""
    cfg = OracleConfig.spec(**CONFIG0)
    e_out, e_attn, e_mlp = _run_block(pkg, cuda, cfg, 0, False, shifted)
    assert e_out <= 1e-2 and e_attn <= 1e-2 and e_mlp <= 1e-2, (e_out, e_attn, e_mlp)


@pytest.mark.parametrize("shifted", [False, True])
def test_config1_block(pkg, cuda, shifted):
    """configs[1]: 180x360 grid, dim 512, 8x64 heads, 12x12 windows (450 windows of 144), shift 6."""
    cfg = OracleConfig.spec(**CONFIG1)
    e_out, e_attn, e_mlp = _run_block(pkg, cuda, cfg, 1, False, shifted)
    assert e_out <= 1e-2 and e_attn <= 1e-2 and e_mlp <= 1e-2, (e_out, e_attn, e_mlp)


@pytest.mark.parametrize("geo", [CONFIG0, SMALL16], ids=["ws8", "ws16"])
@pytest.mark.parametrize("variant", ["spec0", "spec2", "spec3", "ref", "ref_norm_then_mod", "spec_rms_swiglu"])
def test_block_variants_nontrivial(pkg, cuda, geo, variant):
    """Unit-gain weights, non-zero biases / gains / gates (~1): a dropped or misplaced term cannot hide."""
    mk = {"spec0": lambda: OracleConfig.spec(mod_ways=0, **geo), "spec2": lambda: OracleConfig.spec(mod_ways=2, **geo),
          "spec3": lambda: OracleConfig.spec(mod_ways=3, **geo), "ref": lambda: OracleConfig.ref(**geo),
          "ref_norm_then_mod": lambda: OracleConfig.ref(mod_order="norm_then_mod", **geo),
          "spec_rms_swiglu": lambda: OracleConfig.spec(norm="rmsnorm", mlp="swiglu", bias=False, mod_ways=3, **geo)}
    cfg = mk[variant]()
    for shifted in (False, True):
        e_out, e_attn, e_mlp = _run_block(pkg, cuda, cfg, 7, True, shifted, B=2)
        assert e_out <= 1e-2 and e_attn <= 1e-2 and e_mlp <= 1e-2, (variant, shifted, e_out, e_attn, e_mlp)


def test_block_f32_residual_stream(pkg, cuda):
    cfg = OracleConfig.ref(**SMALL16)
    e_out, e_attn, e_mlp = _run_block(pkg, cuda, cfg, 3, True, True, x_dtype=torch.float32, B=2)
    assert e_out <= 6e-3 and e_attn <= 1e-2 and e_mlp <= 1e-2, (e_out, e_attn, e_mlp)


def test_ref_layer_does_not_shift_on_its_own(pkg, cuda):
    """Like the reference's SwinLayer (model.py:368: shifted_grid is ignored), preset "ref" leaves the shift to the model."""
    cfg = OracleConfig.ref(**CONFIG0)
    sd = oracle.init_block_weights(cfg, 5, nontrivial=True)
    layer = pkg.SwinLayer(None, cfg.dim, cfg.heads, cfg.head_dim, cfg.mlp_dim, cfg.window_size, cfg.image_shape, True, 10_000)
    layer.load_state_dict(sd)
    layer = layer.to(torch.bfloat16).to(cuda)
    g = torch.Generator().manual_seed(9)
    x, t = torch.randn(1, 2048, cfg.dim, generator=g).to(torch.bfloat16), torch.randn(1, cfg.dim, generator=g)
    out = layer(x.to(cuda), t.to(cuda))
    assert rel_l2(out, oracle.block_forward(cfg, sd, x.float(), t, (0, 0))) <= 1e-2
    out_s = layer(x.to(cuda), t.to(cuda), shift=(4, 4))
    assert rel_l2(out_s, oracle.block_forward(cfg, sd, x.float(), t, (4, 4))) <= 1e-2
    assert rel_l2(out_s, out) > 1e-2


MODEL_GEO = dict(dim=256, heads=4, head_dim=64, mlp_dim=1024, window_size=(16, 16), image_shape=(32, 64))


@pytest.mark.parametrize("preset,res_dt", [("ref", torch.bfloat16), ("ref", torch.float32), ("spec", torch.bfloat16)])
def test_small_model_parity(pkg, cuda, preset, res_dt):
    """input stage -> 4 blocks (alternating shift) -> output stage, 138 -> 69 channels, with and without APE."""
    mk = OracleConfig.ref if preset == "ref" else (lambda **kw: OracleConfig.spec(mod_ways=2, **kw))
    cfg = mk(n_layers=6, in_channels=138, out_channels=69, **MODEL_GEO)
    for nontrivial in (False, True):
        sd = oracle.init_model_weights(cfg, 11, nontrivial=nontrivial)
        model = make_model(pkg, cfg, sd, cuda, res_dt, preset)
        g = torch.Generator().manual_seed(21)
        B, S = 2, 32 * 64
        x, dt = torch.randn(B, S, 138, generator=g), torch.tensor([0.9])
        ref, ref_h = oracle.model_forward(cfg, sd, x, dt, return_hidden=True)
        out, hid = model(x.to(cuda), dt.to(cuda), return_hidden=True)
        torch.cuda.synchronize()
        assert out.dtype == torch.float32 and out.shape == (B, S, 69)
        assert rel_l2(hid, ref_h) <= 1e-2, (nontrivial, rel_l2(hid, ref_h))
        assert rel_l2(out, ref) <= 1e-2, (nontrivial, rel_l2(out, ref))
        for name, got, want in (("hidden", hid, ref_h), ("output", out, ref)):
            worst = max_abs(got, want) / float(want.double().pow(2).mean().sqrt())
            print(f"small model ({preset}, nontrivial {nontrivial}) {name}: max-abs / rms {worst:.3e}")
            assert worst <= MAX_ABS_OVER_RMS, (name, nontrivial, worst)
    # with the absolute positional encoding of the reference's input stage
    ape = model.generate_ape()
    H, W = cfg.image_shape
    want_ape = oracle.positional_encoding_2d(138, H + 1, W)[1:].reshape(1, H * W, 138)
    assert rel_l2(ape, want_ape) <= 1e-6
    out = model(x.to(cuda), dt.to(cuda))
    ref = oracle.model_forward(cfg, sd, x, dt, ape=want_ape)
    assert rel_l2(out, ref) <= 1e-2


def test_model_output_does_not_depend_on_the_attention_path(pkg, cuda):
    """``Attention.fuse_qkv`` chooses between the to_qkv GEMM + attention kernel pair and the one kernel that keeps
    q, k, v on the chip; both compute the same bits wherever the pair's GEMM is the 256x256-tile kernel (same MFMA shape
    and k order; the grid here is large enough for that), so the whole model's output is bit-identical either way
    (shifted and unshifted blocks, bias table, mask, linear biases, batch 2)."""
    geo = dict(MODEL_GEO, image_shape=(96, 128))
    cfg = OracleConfig.spec(mod_ways=2, n_layers=6, in_channels=138, out_channels=69, **geo)
    assert pkg.ops.gemm_uses_big_tiles(2 * 96 * 128, 3 * cfg.heads * cfg.head_dim)
    sd = oracle.init_model_weights(cfg, 13, nontrivial=True)
    model = make_model(pkg, cfg, sd, cuda, torch.float32, "spec")
    attn = [m for m in model.modules() if isinstance(m, pkg.model.Attention)]
    assert attn and all(m.fuse_qkv == pkg.model.FUSE_QKV_ATTENTION for m in attn)
    assert all(pkg.ops.qkv_attention_supported(cfg.dim, m.heads, m.head_dim, m.window_size, m.image_shape) for m in attn)
    g = torch.Generator().manual_seed(23)
    x, dt = torch.randn(2, 96 * 128, 138, generator=g).to(cuda), torch.tensor([0.7]).to(cuda)
    outs = {}
    for fuse in (True, False):
        for m in attn:
            m.fuse_qkv = fuse
        pkg.ops.profile_begin()
        outs[fuse] = model(x, dt).clone()
        tags = {r[0] for r in pkg.ops.profile_end()}
        assert ("qkv_window_attention" in tags) == fuse and ("window_attention" in tags) == (not fuse), tags
    assert torch.equal(outs[True], outs[False])


def test_reference_window_model_parity(pkg, cuda):
    """The reference's own window geometry (60 x 60 windows of 3600 tokens, head_dim 128, model.py:22-27; preset
    "ref": RMSNorm, 3-way modulation, SwiGLU, no bias / mask) on a 120 x 180 grid: input stage -> 2 layers (the
    second on the half-window-shifted grid) -> output stage, against the oracle."""
    cfg = OracleConfig.ref(n_layers=4, in_channels=138, out_channels=69, dim=256, heads=2, head_dim=128, mlp_dim=512,
                           window_size=(60, 60), image_shape=(120, 180))
    sd = oracle.init_model_weights(cfg, 13, nontrivial=True)
    model = make_model(pkg, cfg, sd, cuda, torch.bfloat16, "ref")
    g = torch.Generator().manual_seed(31)
    x, dt = torch.randn(1, 120 * 180, 138, generator=g), torch.tensor([0.7])
    ref, ref_h = oracle.model_forward(cfg, sd, x, dt, return_hidden=True)
    out, hid = model(x.to(cuda), dt.to(cuda), return_hidden=True)
    torch.cuda.synchronize()
    assert rel_l2(hid, ref_h) <= 1e-2, rel_l2(hid, ref_h)
    assert rel_l2(out, ref) <= 1e-2, rel_l2(out, ref)


def test_sampler_parity_and_graph_replay(pkg, cuda):
    cfg = OracleConfig.ref(n_layers=4, in_channels=24, out_channels=8, dim=128, heads=2, head_dim=64, mlp_dim=256,
                           window_size=(8, 8), image_shape=(16, 24))
    sd = oracle.init_model_weights(cfg, 4, nontrivial=True)
    model = make_model(pkg, cfg, sd, cuda, torch.float32, "ref")
    g = torch.Generator().manual_seed(8)
    B, S = 2, 16 * 24
    cond, lat = torch.randn(B, S, 16, generator=g), torch.randn(B, S, 8, generator=g)
    n = 4
    ref = oracle.sample(lambda m, t: oracle.model_forward(cfg, sd, m, t), cond, lat, oracle.sigma_schedule(n))
    smp = pkg.TrigFlowSampler(model, n_steps=n, device=cuda)
    out = smp.sample(cond.to(cuda), lat.to(cuda))
    torch.cuda.synchronize()
    assert rel_l2(out, ref) <= 1e-2, rel_l2(out, ref)
    # HIP-graph replay: several replays with eager work in between, each equal to the eager result bit for bit
    smp.capture(cond.to(cuda), lat.to(cuda))
    for k in range(3):
        c2, l2 = cond.roll(k, 1).to(cuda), lat.roll(k, 1).to(cuda)
        eager = smp.sample(c2, l2)
        torch.cuda.synchronize()
        replay = smp.sample_graph(c2, l2).clone()
        torch.cuda.synchronize()
        assert torch.equal(eager, replay), k


def test_rollout_parity_eager_and_graph(pkg, cuda):
    """Autoregressive rollout (inference.py:127-186) against the oracle's on the same latents: per-step forcings
    (cat([state, rad_T[k], gp, lsm, rad_T[k+1]]), inference.py:133), non-identity per-channel means / stds for the
    un-standardise / accumulate / re-standardise feedback (era5.py:95-114), two ensemble members as batch; eagerly and
    with the whole forecast step replayed as one HIP graph (bit-identical to eager, also on later replays with eager
    work in between)."""
    C, Cf, Cs, n_fc, n_diff = 8, 3, 2, 3, 3
    cfg = OracleConfig.ref(n_layers=4, in_channels=2 * C + 2 * Cf + Cs, out_channels=C, dim=128, heads=2, head_dim=64,
                           mlp_dim=256, window_size=(8, 8), image_shape=(16, 24))
    sd = oracle.init_model_weights(cfg, 6, nontrivial=True)
    model = make_model(pkg, cfg, sd, cuda, torch.float32, "ref")
    g = torch.Generator().manual_seed(12)
    B, S = 2, 16 * 24
    state0 = torch.randn(B, S, C, generator=g)
    forcing = torch.randn(n_fc + 1, 1, S, Cf, generator=g)
    static = torch.randn(1, S, Cs, generator=g)
    lat = torch.randn(n_fc, B, S, C, generator=g)
    x_mean, x_std = torch.randn(C, generator=g), 0.5 + torch.rand(C, generator=g)
    t_mean, t_std = 0.1 * torch.randn(C, generator=g), 0.2 + 0.2 * torch.rand(C, generator=g)
    kw = dict(x_mean=x_mean, x_std=x_std, t_mean=t_mean, t_std=t_std, forcing=forcing, static=static, latents=lat)
    want = oracle.rollout(lambda m, t: oracle.model_forward(cfg, sd, m, t), state0, n_fc, n_diff, **kw)
    smp = pkg.TrigFlowSampler(model, n_steps=n_diff, device=cuda)
    dkw = {k: v.to(cuda) for k, v in kw.items()}
    eager = smp.rollout(state0.to(cuda), n_fc, **dkw).clone()
    torch.cuda.synchronize()
    assert eager.shape == (n_fc, B, S, C)
    for k in range(n_fc):
        err = rel_l2(eager[k], want[k])
        print(f"rollout step {k}: rel-L2 {err:.3e}, max-abs {max_abs(eager[k], want[k]):.3e}")
        assert err <= 1e-2, (k, err)
    assert rel_l2(eager[1], eager[0]) > 5e-2  # the steps differ: the feedback and the per-step forcings are live
    ro = smp.begin_rollout(state0.to(cuda), n_fc, use_graph=True, graph_warmup=1, **dkw)
    graph = ro.run().clone()
    torch.cuda.synchronize()
    assert torch.equal(graph, eager)
    ro.reset()
    for k in range(n_fc):  # replays with eager kernels and a synchronisation in between
        ro.run(1)
        model(torch.randn(B, S, cfg.in_channels, device=cuda), torch.tensor([0.3], device=cuda))
        torch.cuda.synchronize()
        assert torch.equal(ro.states[k], eager[k]), k
    # the whole rollout as ONE graph and one replay (the step counter, forcings and state store are indexed on the device)
    whole = smp.begin_rollout(state0.to(cuda), n_fc, use_graph=True, graph_steps=n_fc, **dkw)
    assert torch.equal(whole.run(), eager)
    whole.reset()
    model(torch.randn(B, S, cfg.in_channels, device=cuda), torch.tensor([0.7], device=cuda))  # eager work in between
    assert torch.equal(whole.run(), eager)
    with pytest.raises(ValueError, match="multiple"):
        whole.reset()
        whole.run(1)
    # a generator instead of given latents: the graph draws its latents on the device, every replay new ones
    gen = torch.Generator(device="cuda").manual_seed(3)
    drawn = smp.rollout(state0.to(cuda), 2, gen, use_graph=True, **{k: v for k, v in dkw.items() if k != "latents"})
    torch.cuda.synchronize()
    assert bool(torch.isfinite(drawn).all()) and rel_l2(drawn[1], drawn[0]) > 5e-2
    # a seeded rollout gives the same forecast eagerly and replayed, although the graph path first runs a warm-up step
    # that draws latents too (the generator is put back), and although work is still pending on the main stream when
    # the warm-up moves to its side stream (the shared block intermediates change hands without an error)
    nolat = {k: v for k, v in dkw.items() if k != "latents"}
    e_seeded = smp.rollout(state0.to(cuda), 2, torch.Generator(device="cuda").manual_seed(3), **nolat).clone()
    busy = torch.randn(64, 1024, 1024, device=cuda)
    for _ in range(30):
        busy = busy * 1.0001  # queued on the main stream, not waited for
    model(torch.randn(B, S, cfg.in_channels, device=cuda), torch.tensor([0.3], device=cuda))  # main stream owns the scratch
    g_seeded = smp.rollout(state0.to(cuda), 2, torch.Generator(device="cuda").manual_seed(3), use_graph=True,
                           graph_warmup=1, **nolat)
    torch.cuda.synchronize()
    assert torch.equal(g_seeded, e_seeded)


@pytest.mark.parametrize("name,geo", [("config2", dict(dim=1024, heads=16, head_dim=64, mlp_dim=4096)),
                                      ("config3", dict(dim=1536, heads=24, head_dim=64, mlp_dim=6144))])
def test_full_grid_block_against_oracle_strips(pkg, cuda, name, geo):
    """Full 720x1440 grid (1 036 800 tokens, 4 050 windows of 16x16).  A Swin block only mixes tokens inside one
    window, so a band of window rows of the full-grid result must equal the oracle run on that band alone: rows
    [16k, 16k+16) for the un-shifted block; rows [16k+8, 16k+24) with a longitude-only shift for the shifted block
    (no latitude wrap inside the band); the last band of the shifted block wraps in latitude (rows 712..719 + 0..7)
    and carries the full shift mask."""
    H, W, ws = 720, 1440, 16
    cfg = OracleConfig.spec(window_size=(ws, ws), image_shape=(H, W), mod_ways=2, **geo)
    sd = oracle.init_block_weights(cfg, 17, nontrivial=True)
    g = torch.Generator(device="cuda").manual_seed(5)
    x = torch.randn(1, H * W, cfg.dim, generator=g, device=cuda, dtype=torch.float32).to(torch.bfloat16)
    t = torch.randn(1, cfg.dim, generator=torch.Generator().manual_seed(6))
    for shifted in (False, True):
        layer = make_layer(pkg, cfg, sd, cuda, shifted)
        out = layer(x, t.to(cuda))
        out2 = layer(x, t.to(cuda))
        torch.cuda.synchronize()
        assert torch.equal(out, out2)  # deterministic
        grid_in = x.view(H, W, cfg.dim)
        grid_out = out.view(H, W, cfg.dim)
        bands = [0, 22, 44] if not shifted else [0, 21, 44]
        for k in bands:
            if not shifted:
                rows = torch.arange(16 * k, 16 * k + 16)
                band_cfg = OracleConfig.spec(window_size=(ws, ws), image_shape=(16, W), mod_ways=2, **geo)
                shift = (0, 0)
            elif k < 44:
                rows = torch.arange(16 * k + 8, 16 * k + 24)
                band_cfg = OracleConfig.spec(window_size=(ws, ws), image_shape=(16, W), mod_ways=2, **geo)
                shift = (0, 8)
            else:  # wrapped band: rows 0..23 followed by rows 712..719 form a 32-row image whose half-window roll puts
                #    rows 8..23 into its first window row and rows 712..719 + 0..7 into its last, masked, window row:
                #    exactly the first and the last window row of the rolled full grid
                rows = torch.cat([torch.arange(0, 24), torch.arange(712, 720)])
                band_cfg = OracleConfig.spec(window_size=(ws, ws), image_shape=(32, W), mod_ways=2, **geo)
                shift = (8, 8)
            xin = grid_in[rows.to(cuda)].float().cpu().reshape(1, -1, cfg.dim)
            ref = oracle.block_forward(band_cfg, sd, xin, t, shift).reshape(len(rows), W, cfg.dim)
            got = grid_out[rows.to(cuda)].float().cpu()
            err = rel_l2(got, ref)
            assert err <= 1e-2, (name, shifted, k, err)


def test_full_grid_ensemble_batch_matches_single_members(pkg, cuda):
    """configs[4] shape: 4 ensemble members as batch 4 on the 720x1440 grid (4 147 200 rows through every kernel,
    per-member modulation vectors).  A member's rows of the batched result must be bit-identical to running that
    member alone: windows, GEMM tiles (1 036 800 = 4050 x 256 rows per member) and norm rows never mix members."""
    H, W, ws = 720, 1440, 16
    cfg = OracleConfig.spec(window_size=(ws, ws), image_shape=(H, W), mod_ways=2, dim=1536, heads=24, head_dim=64,
                            mlp_dim=6144)
    sd = oracle.init_block_weights(cfg, 23, nontrivial=True)
    g = torch.Generator(device="cuda").manual_seed(9)
    x = torch.randn(4, H * W, cfg.dim, generator=g, device=cuda, dtype=torch.float32).to(torch.bfloat16)
    t = torch.randn(4, cfg.dim, generator=torch.Generator().manual_seed(10)).to(cuda)
    for shifted in (False, True):
        layer = make_layer(pkg, cfg, sd, cuda, shifted)
        out = layer(x, t).clone()
        for b in (0, 3):
            single = layer(x[b:b + 1].contiguous(), t[b:b + 1].contiguous())
            torch.cuda.synchronize()
            assert torch.equal(out[b:b + 1], single), (shifted, b)
        assert bool(torch.isfinite(out.float()).all())


def test_full_size_ensemble_rollout_graph_matches_eager(pkg, cuda):
    """configs[4] at its full size: the configs[3] denoiser (24 blocks, dim 1536, 24 x 64 heads, 16x16 windows) on the
    720x1440 grid with 4 ensemble members as batch 4, two autoregressive forecast steps of a 2-step Heun sampler (3
    denoiser calls each, inference.py:136-186), the forecast step captured as one HIP graph.  The replayed rollout must
    equal the eager one bit for bit, every state must be finite, and member 0 of the batch must be bit for bit the
    forecast of that member run alone (windows, GEMM tiles and norm rows never mix members)."""
    import bench
    wl = bench.WORKLOADS["config4"]
    H, W = wl["image_shape"]
    S, B, C, n_fc = H * W, 4, wl["cout"], 2
    model = bench.build_model(pkg, torch, wl, cuda, torch.float32)
    g = torch.Generator(device="cuda").manual_seed(4)
    state0 = torch.randn(B, S, C, generator=g, device=cuda)
    lat = torch.randn(n_fc, B, S, C, generator=g, device=cuda)
    smp = pkg.TrigFlowSampler(model, n_steps=2, device=cuda)
    print("full-size rollout: eager", flush=True)
    eager = smp.rollout(state0, n_fc, latents=lat).clone()
    torch.cuda.synchronize()
    assert eager.shape == (n_fc, B, S, C) and bool(torch.isfinite(eager).all())
    assert rel_l2(eager[1], eager[0]) > 1e-3  # the second step starts from the first step's state
    print("full-size rollout: graph", flush=True)
    ro = smp.begin_rollout(state0, n_fc, latents=lat, use_graph=True)
    replayed = ro.run()
    torch.cuda.synchronize()
    assert torch.equal(replayed, eager)
    del ro, replayed
    print("full-size rollout: member 0 alone", flush=True)
    alone = smp.rollout(state0[:1].contiguous(), n_fc, latents=lat[:, :1].contiguous())
    torch.cuda.synchronize()
    assert torch.equal(alone[:, 0], eager[:, 0])


@pytest.mark.gpu
def test_bench_json_contract_on_a_small_workload(pkg, cuda, monkeypatch, capsys):
    """bench.py's one JSON line carries the fields its callers read (run in-process on the configs[1] shape: seconds)."""
    import json
    import sys
    import bench
    monkeypatch.setattr(sys, "argv", ["bench.py", "--workload", "config1", "--steps", "1", "--warmup", "0", "--cpu-rows", "12"])
    bench.main()
    line = [l for l in capsys.readouterr().out.strip().splitlines() if l.startswith("{")][-1]
    r = json.loads(line)
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "roofline", "kernels", "cpu_baseline", "parity"):
        assert key in r, key
    assert r["n_gpus"] == 1 and r["steps"] == 1 and r["higher_is_better"] is True and r["vs_baseline"] is None
    assert r["value"] > 0 and abs(r["value"] * r["ms_per_step"] - 1000.0) < 1e-6 * 1000.0
    assert "workload" in r["config"] and "model" not in r["config"]
    assert r["output_finite"] is True
    assert r["parity"]["rel_l2"] <= 1e-2 and r["parity"]["max_abs"] > 0  # the timed model against the oracle, full depth
    cb = r["cpu_baseline"]
    assert cb["kind"] == "port" and cb["cores"] >= 1 and cb["value"] > 0 and "sample" in cb
    if r["roofline"] is not None:
        rf = r["roofline"]
        assert rf["bound"] in ("hbm", "mfma") and abs(rf["frac"] - rf["achieved"] / rf["peak"]) < 1e-9
    for k in r["kernels"].values():
        assert k["launches_per_step"] >= 1 and k["avg_ms"] > 0
