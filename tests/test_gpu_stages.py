"""GPU parity of the pieces around the Swin blocks, each on its own: input stage, output stage, the checkpoint
converter feeding the GPU model, and the guards of the shared scratch buffers and of the lazy initialisation.

The reference keeps both stages in fp32 (model.py:350-352, 422-428); their errors are reported as relative L2 and
max-abs against the fp32 oracle.
"""
import os
import subprocess
import sys
import textwrap

import pytest
import torch

import oracle
from oracle import OracleConfig
from helpers import make_model, rel_l2, max_abs

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
GEO = dict(dim=1536, heads=24, head_dim=64, mlp_dim=256, window_size=(16, 16), image_shape=(32, 64))


def _stage_model(pkg, cuda, preset, nontrivial=True):
    mk = OracleConfig.ref if preset == "ref" else (lambda **kw: OracleConfig.spec(mod_ways=2, **kw))
    cfg = mk(n_layers=2, in_channels=138, out_channels=69, **GEO)  # n_layers = 2: no Swin layer, the two stages only
    sd = oracle.init_model_weights(cfg, 2, nontrivial=nontrivial)
    return cfg, sd, make_model(pkg, cfg, sd, cuda, torch.float32, preset)


@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16], ids=["f32_tokens", "bf16_tokens"])
def test_input_stage_alone(pkg, cuda, out_dtype):
    """(+APE) -> Linear(138 -> 1536) + bias, and the noise-level embedding (model.py:346-356); plain input, the
    sampler's [x / sigma_d | cond] concatenation folded into the operand, and with the positional encoding."""
    cfg, sd, model = _stage_model(pkg, cuda, "ref")
    g = torch.Generator().manual_seed(3)
    B, S = 2, 32 * 64
    x, dt = torch.randn(B, S, 138, generator=g), torch.tensor([1.1])
    want, want_t = oracle.input_stage(cfg, sd, x, dt)
    tok, t = model.input_stage(x.to(cuda), dt.to(cuda), out_dtype=out_dtype)
    torch.cuda.synchronize()
    bound = 2e-5 if out_dtype == torch.float32 else 3e-3  # f32 tokens: the reference's fp32 Linear; bf16: one rounding
    e = rel_l2(tok, want)
    print(f"input stage ({out_dtype}): rel-L2 {e:.3e}, max-abs {max_abs(tok, want):.3e}; t embedding {rel_l2(t, want_t):.2e}")
    assert tok.dtype == out_dtype and e <= bound, e
    assert rel_l2(t, want_t) <= 1e-5
    # concatenation folded into the operand: [x0 / 2 | x1]
    x0, x1 = x[..., :69].contiguous(), x[..., 69:].contiguous()
    tok2, _ = model.input_stage(x0.to(cuda), dt.to(cuda), out_dtype=out_dtype, cond=x1.to(cuda), x_div=2.0)
    want2, _ = oracle.input_stage(cfg, sd, torch.cat([x0 / 2.0, x1], dim=2), dt)
    assert rel_l2(tok2, want2) <= bound, rel_l2(tok2, want2)
    # absolute positional encoding added to the input channels (model.py:350)
    ape = model.generate_ape()
    want_ape = oracle.positional_encoding_2d(138, 33, 64)[1:].reshape(1, S, 138)
    tok3, _ = model.input_stage(x.to(cuda), dt.to(cuda), out_dtype=out_dtype)
    want3, _ = oracle.input_stage(cfg, sd, x, dt, ape=want_ape)
    assert rel_l2(tok3, want3) <= bound, rel_l2(tok3, want3)
    assert rel_l2(tok3, want) > 1e-2  # the encoding is live


@pytest.mark.parametrize("case", [
    # (M, M_ape, C0, C1, d, div0, bias, out dtype)
    (4096, 2048, 69, 69, 1536, 0.5, True, torch.float32),    # the sampler's form, two batch entries share the encoding
    (2048, 2048, 138, 0, 1536, 1.0, True, torch.bfloat16),   # plain input, bf16 tokens
    (1000, 0, 20, 11, 256, 2.0, True, torch.float32),        # ragged rows (1000 = 3 x 256 + 232), one k-step, no encoding
    (777, 259, 40, 23, 64, 1.0, False, torch.float32),       # encoding wraps inside a workgroup, no bias, two k-steps
    (300, 100, 96, 0, 128, 3.0, True, torch.float32),        # C = 96: the bias column opens a fourth k-step
    (256, 256, 159, 0, 192, 1.0, True, torch.float32),       # the widest input the kernel takes
], ids=["sampler", "plain_bf16", "ragged_small", "wrap_nobias", "k96", "k159"])
def test_input_stage_kernel_against_float64(pkg, cuda, case):
    """ops.input_stage (one kernel: channel concatenation, division, positional encoding, Linear + bias) against the
    same arithmetic in float64.  The reference computes this Linear in fp32 (model.py:350-352)."""
    M, M_ape, C0, C1, d, div0, with_bias, out_dtype = case
    ops = pkg.ops
    g = torch.Generator().manual_seed(M + d)
    C = C0 + C1
    x0 = torch.randn(M, C0, generator=g) * 3.0
    x1 = torch.randn(M, C1, generator=g) if C1 else None
    ape = torch.rand(M_ape, C, generator=g) * 2.0 - 1.0 if M_ape else None
    w = torch.randn(d, C, generator=g) * 0.1
    b = torch.randn(d, generator=g) if with_bias else None
    assert ops.input_stage_supported(C, d)
    packed = ops.input_stage_pack_weight(w.to(cuda), None if b is None else b.to(cuda))
    got = ops.input_stage(x0.to(cuda), div0, None if x1 is None else x1.to(cuda), None if ape is None else ape.to(cuda),
                          packed, d, out_dtype=out_dtype)
    torch.cuda.synchronize()
    xin = (x0 / div0).double()
    if x1 is not None:
        xin = torch.cat([xin, x1.double()], dim=1)
    if ape is not None:
        xin = xin + ape.double().repeat(-(-M // M_ape), 1)[:M]
    want = xin @ w.double().t() + (0 if b is None else b.double())
    e, ma = rel_l2(got, want), max_abs(got, want)
    print(f"input stage kernel {case[:5]}: rel-L2 {e:.3e}, max-abs {ma:.3e}")
    assert got.dtype == out_dtype and tuple(got.shape) == (M, d)
    assert e <= (1e-5 if out_dtype == torch.float32 else 3e-3), (e, ma)


def test_input_stage_without_encoding_keeps_a_non_finite_input_in_its_own_token(pkg, cuda):
    """No positional encoding: an Inf (or NaN) in the first element of the input makes token 0 non-finite, as in the
    reference's Linear, and leaves every other token exactly what it is with a finite value there."""
    ops = pkg.ops
    M, C0, C1, d = 600, 20, 11, 256
    g = torch.Generator().manual_seed(3)
    x0, x1 = torch.randn(M, C0, generator=g), torch.randn(M, C1, generator=g)
    w, b = torch.randn(d, C0 + C1, generator=g) * 0.1, torch.randn(d, generator=g)
    packed = ops.input_stage_pack_weight(w.to(cuda), b.to(cuda))
    clean = ops.input_stage(x0.to(cuda), 2.0, x1.to(cuda), None, packed, d).clone()
    for bad in (float("inf"), float("nan")):
        x0b = x0.clone()
        x0b[0, 0] = bad
        got = ops.input_stage(x0b.to(cuda), 2.0, x1.to(cuda), None, packed, d)
        torch.cuda.synchronize()
        assert not bool(torch.isfinite(got[0]).all())
        assert torch.equal(got[1:], clean[1:])


def test_input_stage_falls_back_for_wide_inputs(pkg, cuda):
    """More than 159 input channels: the operand-matrix + GEMM form, same accuracy."""
    ops = pkg.ops
    assert not ops.input_stage_supported(200, 256) and not ops.input_stage_supported(64, 200)
    stage = pkg.InputStage(200, 256, 10000.0).to(cuda)
    g = torch.Generator().manual_seed(5)
    x = torch.randn(1, 512, 200, generator=g)
    tok, _ = stage(x.to(cuda), torch.tensor([0.3], device=cuda), out_dtype=torch.float32)
    want = x.double() @ stage.proj.weight.detach().double().cpu().t() + stage.proj.bias.detach().double().cpu()
    assert rel_l2(tok, want) <= 2e-5, rel_l2(tok, want)


@pytest.mark.parametrize("preset", ["ref", "spec"])
@pytest.mark.parametrize("x_dtype", [torch.float32, torch.bfloat16], ids=["f32_stream", "bf16_stream"])
def test_output_stage_alone(pkg, cuda, preset, x_dtype):
    """norm -> modulate(shift, scale) -> head (model.py:421-429), fp32 in the reference."""
    cfg, sd, model = _stage_model(pkg, cuda, preset)
    g = torch.Generator().manual_seed(4)
    B, S = 2, 32 * 64
    x = (2.0 * torch.randn(B, S, cfg.dim, generator=g) + 0.3).to(x_dtype)
    t_emb = oracle.timestep_embedding(torch.tensor([0.4]), cfg.dim)
    want = oracle.output_stage(cfg, sd, x.float(), t_emb)
    out = model.output_stage(x.to(cuda), t_emb.to(cuda))
    torch.cuda.synchronize()
    e = rel_l2(out, want)
    print(f"output stage ({preset}, {x_dtype}): rel-L2 {e:.3e}, max-abs {max_abs(out, want):.3e}")
    assert out.dtype == torch.float32 and out.shape == (B, S, 69)
    assert e <= 2e-5, e


@pytest.mark.parametrize("case", [
    # B, S, d, N, kind, x dtype, modulation rows, row mean
    (1, 1000, 1536, 69, "layernorm", torch.float32, 1, 0.0),    # ragged row count (1000 = 15 tiles + 40 rows)
    (3, 128, 1536, 70, "rmsnorm", torch.float32, 3, 0.0),       # one modulation row per batch entry
    (2, 192, 256, 8, "layernorm", torch.bfloat16, 2, 0.0),      # one column fragment, bf16 tokens
    (1, 4096, 1024, 80, "layernorm", torch.float32, 0, 0.0),    # no modulation at all, five full fragments
    (1, 640, 1536, 69, "layernorm", torch.float32, 1, 100.0),   # rows with |mean| = 50 sigma: the provisional centre
    (2, 100, 128, 33, "rmsnorm", torch.bfloat16, 1, 3.0),
], ids=lambda c: f"B{c[0]}_S{c[1]}_d{c[2]}_N{c[3]}_{c[4]}_{'f32' if c[5] == torch.float32 else 'bf16'}_mod{c[6]}_mean{c[7]:g}")
def test_output_stage_kernel_against_float64(pkg, cuda, case):
    """aeris_output_stage_fwd against norm -> modulate -> Linear evaluated in float64 (torch.nn.functional)."""
    B, S, d, N, kind, x_dt, mod_rows, mean = case
    g = torch.Generator().manual_seed(B * 1000 + S + d + N)
    x = (2.0 * torch.randn(B, S, d, generator=g) + mean * (1 + torch.rand(B, S, 1, generator=g))).to(x_dt)
    gamma, beta = 1 + 0.2 * torch.randn(d, generator=g), 0.3 * torch.randn(d, generator=g)
    w = torch.randn(N, d, generator=g) / d ** 0.5
    m = 0.3 * torch.randn(max(mod_rows, 1), 2 * d, generator=g)
    shift, scale = (m[:, :d], m[:, d:]) if mod_rows else (None, None)
    xd = x.double()
    if kind == "layernorm":
        y = torch.nn.functional.layer_norm(xd, (d,), gamma.double(), beta.double(), 1e-5)
    else:
        y = torch.nn.functional.rms_norm(xd, (d,), gamma.double(), 1e-6)
    if mod_rows:
        y = y * (1 + scale.double().unsqueeze(1)) + shift.double().unsqueeze(1)
    want = y @ w.double().T
    dev = lambda t: None if t is None else t.to(cuda)
    md = m.to(cuda)
    out = pkg.ops.output_stage(dev(x), dev(gamma), dev(beta) if kind == "layernorm" else None,
                               md[:, :d] if mod_rows else None, md[:, d:] if mod_rows else None, dev(w), kind=kind,
                               eps=1e-5 if kind == "layernorm" else 1e-6)
    torch.cuda.synchronize()
    e = rel_l2(out, want)
    print(f"fused output stage {case[:5]}: rel-L2 {e:.3e}, max-abs {max_abs(out, want):.3e}")
    assert out.shape == (B, S, N) and e <= (2e-5 if mean < 50 else 2e-4), e


def test_converted_checkpoint_runs_on_the_gpu(pkg, cuda, tmp_path):
    """convert_inference_checkpoint (model.py:479-495) straight onto the device: per-pipeline-stage ``ema_state_dict``
    files, including the stray ``latent_embed`` / ``1.norm`` entries the reference drops, are stitched into the model,
    which then runs with the generated positional encoding (inference.py:281-297) and matches the oracle."""
    cfg = OracleConfig.ref(n_layers=5, sublayers=2, in_channels=144, out_channels=70, dim=256, heads=2, head_dim=128,
                           mlp_dim=512, window_size=(12, 8), image_shape=(24, 32))
    sd = oracle.init_model_weights(cfg, 9, nontrivial=True)
    N = cfg.n_layers
    stages = [dict() for _ in range(N)]
    for k, v in sd.items():
        if k.startswith("input_stage."):
            stages[0][k[len("input_stage."):]] = v
        elif k.startswith("output_stage."):
            stages[N - 1][k[len("output_stage."):]] = v
        else:
            _, i, rest = k.split(".", 2)
            stages[int(i) + 1][rest] = v.to(torch.bfloat16)  # the trainer's layers are bf16
    stages[0]["ape.inv_freq"] = pkg.PositionalEncoding2D(144).inv_freq.clone()
    stages[0]["latent_embed.weight"] = torch.zeros(3, 3)
    stages[1]["modulelist.1.norm.weight"] = torch.zeros(3)
    for k, st in enumerate(stages):
        torch.save({"ema_state_dict": st, "iteration": 7}, tmp_path / f"checkpoint_PP{k}.pth")
    model = pkg.LocalAERIS(device_mesh=None, heads=cfg.heads, dim=cfg.dim, head_dim=cfg.head_dim, mlp_dim=cfg.mlp_dim,
                           window_size=cfg.window_size, image_shape=cfg.image_shape, rope_base=10_000, sublayers=cfg.sublayers,
                           sinusoidal_emb_max_period=cfg.max_period, n_layers=N, model_in_channels=144,
                           model_out_channels=70).to(cuda)
    pkg.convert_inference_checkpoint(str(tmp_path), N, model, map_location="cuda")
    assert all(p.is_cuda for p in model.parameters())
    assert model.layers[0].modulelist[1][1].to_qkv.weight.dtype == torch.bfloat16
    ape = model.generate_ape()
    H, W = cfg.image_shape
    want_ape = oracle.positional_encoding_2d(144, H + 1, W)[1:].reshape(1, H * W, 144)
    assert rel_l2(ape, want_ape) <= 1e-6
    g = torch.Generator().manual_seed(5)
    x, dt = torch.randn(1, H * W, 144, generator=g), torch.tensor([0.6])
    sd_bf = {k: (v.to(torch.bfloat16).float() if k.startswith("layers.") else v) for k, v in sd.items()}
    want = oracle.model_forward(cfg, sd_bf, x, dt, ape=want_ape)
    out = model(x.to(cuda), dt.to(cuda))
    torch.cuda.synchronize()
    e = rel_l2(out, want)
    print(f"converted checkpoint: rel-L2 {e:.3e}, max-abs {max_abs(out, want):.3e}")
    assert e <= 1e-2, e
    # a checkpoint that does not match the model 1:1 is refused (the reference asserts key-set equality, model.py:494)
    torch.save({"ema_state_dict": {k: v for k, v in stages[2].items() if "wo" not in k}}, tmp_path / "checkpoint_PP2.pth")
    with pytest.raises(KeyError):
        pkg.convert_inference_checkpoint(str(tmp_path), N, model, map_location="cuda")


def test_workspace_refuses_a_second_stream_while_the_first_is_busy(pkg, cuda):
    """The block intermediates are one set of scratch buffers per device; a second stream asking for them while the
    first still has work pending would overwrite them under that work, so the request raises.  Once the first stream
    has drained the buffers change hands."""
    cfg = OracleConfig.spec(dim=1024, heads=16, head_dim=64, mlp_dim=4096, window_size=(16, 16), image_shape=(256, 512),
                            mod_ways=0)
    sd = oracle.init_block_weights(cfg, 1)
    from helpers import make_layer
    layer = make_layer(pkg, cfg, sd, cuda, False)
    x = torch.randn(1, 256 * 512, 1024, device=cuda).to(torch.bfloat16)
    layer(x)
    torch.cuda.synchronize()
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
    with torch.cuda.stream(s1):
        for _ in range(4):  # tens of milliseconds of queued work
            y1 = layer(x)
    with torch.cuda.stream(s2):
        with pytest.raises(RuntimeError, match="another stream"):
            layer(x)
    torch.cuda.synchronize()
    with torch.cuda.stream(s2):  # the first stream is idle now
        y2 = layer(x)
    torch.cuda.synchronize()
    assert torch.equal(y1, y2)


def test_first_call_inside_a_capture_is_refused():
    """Kernel attributes are configured once per process, outside any stream capture: a launch entry point that finds
    the library uninitialised on a capturing stream returns AERIS_EINVAL instead of configuring inside the capture.
    Needs a process in which aeris_init has not run, hence the child process."""
    code = textwrap.dedent("""
        import importlib, sys, torch
        sys.path.insert(0, %r)
        pkg = importlib.import_module("aeris-gb_amd")
        dev = torch.device("cuda:0")
        a = torch.zeros(256, 64, dtype=torch.bfloat16, device=dev)
        w = torch.zeros(256, 64, dtype=torch.bfloat16, device=dev)
        out = torch.empty(256, 256, dtype=torch.bfloat16, device=dev)
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        msg = ""
        try:
            with torch.cuda.graph(g):
                try:
                    pkg.ops.gemm(a, w, out=out)
                except RuntimeError as e:
                    msg = str(e)
        except RuntimeError:
            pass
        assert "aeris_init" in msg, msg
        pkg._lib.call("aeris_init")
        g2 = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g2):
            pkg.ops.gemm(a, w, out=out)
        g2.replay()
        torch.cuda.synchronize()
        print("CHILD_OK")
    """ % ROOT)
    r = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, timeout=150)
    assert "CHILD_OK" in r.stdout, (r.stdout[-2000:], r.stderr[-2000:])
