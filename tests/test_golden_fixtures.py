"""The committed fixture tests/golden/swin_block_small.npz (built from library routines and explicit loops by
tests/golden/make_golden.py, without oracle/ arithmetic) against the oracle on the CPU and against the HIP path."""
import os

import numpy as np
import pytest
import torch

import oracle
from helpers import make_layer, rel_l2

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
    out = layer(x, torch.from_numpy(z["t_emb"]).to(cuda), branches=branches)
    torch.cuda.synchronize()
    assert rel_l2(out, torch.from_numpy(z["out"])) <= 1e-2
    assert rel_l2(branches["attn"], torch.from_numpy(z["attn_branch"])) <= 1e-2
    assert rel_l2(branches["mlp"], torch.from_numpy(z["mlp_branch"])) <= 1e-2
