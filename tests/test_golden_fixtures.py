"""The committed fixture tests/golden/swin_block_small.npz (built from library routines and explicit loops by
tests/golden/make_golden.py, without oracle/ arithmetic) against the oracle on the CPU and against the HIP path."""
import os

import numpy as np
import pytest
import torch

import oracle
from helpers import branch_tap, make_layer, rel_l2

FIX = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "swin_block_small.npz")


def _load():
    z = np.load(FIX, allow_pickle=False)
    H, W, ws, s, dim, heads, hd, mlp, seed = (int(v) for v in z["geometry"])
    cfg = oracle.OracleConfig.spec(dim=dim, heads=heads, head_dim=hd, mlp_dim=mlp, window_size=(ws, ws), image_shape=(H, W),
                                   mod_ways=2)
    return z, cfg, (H, W, ws, s), oracle.init_block_weights(cfg, seed, nontrivial=True)


def test_oracle_integer_maps_match_fixture():
    z, cfg, (H, W, ws, s), _ = _load()
    np.testing.assert_array_equal(oracle.window_token_index(1, H, W, ws, ws, s, s), z["window_token_index"])
    np.testing.assert_array_equal(oracle.relative_position_index(ws, ws), z["relative_position_index"])
    np.testing.assert_array_equal(oracle.shift_attention_mask(H, W, ws, ws, s, s), z["shift_mask"])


def test_oracle_block_matches_fixture():
    z, cfg, (H, W, ws, s), sd = _load()
    out, attn, mlp = oracle.block_forward(cfg, sd, torch.from_numpy(z["x"]), torch.from_numpy(z["t_emb"]), (s, s),
                                          return_branches=True)
    for got, key in ((out, "out"), (attn, "attn_branch"), (mlp, "mlp_branch")):
        assert rel_l2(got, torch.from_numpy(z[key])) <= 2e-6, key  # fp32 oracle vs float64 library composition


@pytest.mark.gpu
def test_hip_block_matches_fixture(pkg, cuda):
    z, cfg, (H, W, ws, s), sd = _load()
    layer = make_layer(pkg, cfg, sd, cuda, shifted=True)
    branches = {}
    x = torch.from_numpy(z["x"]).to(torch.bfloat16).to(cuda)
    out = layer(x, torch.from_numpy(z["t_emb"]).to(cuda), tap=branch_tap(pkg, branches))
    torch.cuda.synchronize()
    assert rel_l2(out, torch.from_numpy(z["out"])) <= 1e-2
    assert rel_l2(branches["attn"].view(z["attn_branch"].shape), torch.from_numpy(z["attn_branch"])) <= 1e-2
    assert rel_l2(branches["mlp"].view(z["mlp_branch"].shape), torch.from_numpy(z["mlp_branch"])) <= 1e-2


# ---- the reference's own block form (model.py: RMSNorm, modulation before the norm, gates, SwiGLU, no biases), un-shifted and
# between the two model-level shifts: tests/golden/ref_block_small.npz, built by tests/golden/make_golden_ref.py
REF_FIX = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "ref_block_small.npz")


def _load_ref():
    z = np.load(REF_FIX, allow_pickle=False)
    H, W, wy, wx, dim, heads, hd, mlp, seed = (int(v) for v in z["geometry"])
    cfg = oracle.OracleConfig.ref(dim=dim, heads=heads, head_dim=hd, mlp_dim=mlp, window_size=(wy, wx), image_shape=(H, W))
    return z, cfg, oracle.init_block_weights(cfg, seed, nontrivial=True)


def test_oracle_ref_block_matches_fixture():
    z, cfg, sd = _load_ref()
    x, t = torch.from_numpy(z["x"]), torch.from_numpy(z["t_emb"])
    wy, wx = cfg.window_size
    assert rel_l2(oracle.block_forward(cfg, sd, x, t, (0, 0)), torch.from_numpy(z["out_plain"])) <= 2e-6
    # shift folded into the attention addressing == roll, layer, roll back (model.py:471-475)
    assert rel_l2(oracle.block_forward(cfg, sd, x, t, (wy // 2, wx // 2)), torch.from_numpy(z["out_shifted"])) <= 2e-6
    assert rel_l2(torch.from_numpy(z["out_plain"]), torch.from_numpy(z["out_shifted"])) > 1e-2  # the shift matters here


@pytest.mark.gpu
def test_hip_ref_layers_match_fixture(pkg, cuda):
    """The reference preset's SwinLayer on the fixture input: un-shifted, between swin_shift up and down as
    model.py:469-475 runs odd layers, and with the shift folded into the attention kernel as LocalAERIS here runs them."""
    z, cfg, sd = _load_ref()
    x = torch.from_numpy(z["x"]).to(torch.bfloat16).to(cuda)
    t = torch.from_numpy(z["t_emb"]).to(cuda)
    layer = pkg.SwinLayer(None, cfg.dim, cfg.heads, cfg.head_dim, cfg.mlp_dim, cfg.window_size, cfg.image_shape, False, 10_000,
                          preset="ref")
    layer.load_state_dict(sd, strict=True)
    layer = layer.to(torch.bfloat16).to(cuda)
    out = layer(x, t)
    up = pkg.swin_shift(x, True, img_shape=cfg.image_shape, window_size=cfg.window_size)
    out_s = pkg.swin_shift(layer(up, t), False, img_shape=cfg.image_shape, window_size=cfg.window_size)
    # what LocalAERIS does for odd layers instead: no rolled copies, the shift folded into the attention addresses
    wy, wx = cfg.window_size
    out_f = layer(x, t, shift=(wy // 2, wx // 2))
    torch.cuda.synchronize()
    assert rel_l2(out, torch.from_numpy(z["out_plain"])) <= 1e-2
    assert rel_l2(out_s, torch.from_numpy(z["out_shifted"])) <= 1e-2
    assert rel_l2(out_f, torch.from_numpy(z["out_shifted"])) <= 1e-2
    assert torch.equal(out_f, out_s)  # index maps are exact: folding the shift changes no bit
