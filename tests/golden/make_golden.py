"""Writes tests/golden/swin_block_small.npz: inputs and expected outputs of one shifted Swin block of the benchmark kind
(LayerNorm, scale/shift modulation after the norm, relative-position bias, shift mask, GELU MLP, biases) and the integer
maps of a small grid.

The reference (src/aeris_wp_inference) ships no tests or vectors and was not run.  The expected values here are built
from library routines and from the textbook shifted-window recipe written out with explicit loops - torch.roll,
einops.rearrange, F.layer_norm, F.scaled_dot_product_attention, F.gelu, F.linear, F.silu - and NOT with any function of
oracle/: the fixture pins the oracle (tests/test_golden_fixtures.py) from the outside.  Only the seeded weights come from
oracle.init_block_weights (data, not arithmetic).

    python tests/golden/make_golden.py        # rewrites the .npz next to this file
"""
import os
import sys

import numpy as np
import torch
import torch.nn.functional as F
from einops import rearrange

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
import oracle  # noqa: E402  (weights only)

H, W, WS, SHIFT = 16, 16, 8, 4
DIM, HEADS, HD, MLP = 64, 2, 32, 256
SEED = 5


def relative_position_index_loops(ws):
    idx = np.zeros((ws * ws, ws * ws), dtype=np.int64)
    for qy in range(ws):
        for qx in range(ws):
            for ky in range(ws):
                for kx in range(ws):
                    idx[qy * ws + qx, ky * ws + kx] = (qy - ky + ws - 1) * (2 * ws - 1) + (qx - kx + ws - 1)
    return idx


def shift_mask_loops(H, W, ws, s):
    """-100 between tokens of one window that come from different sides of the wrapped border (Swin's img_mask)."""
    region = np.zeros((H, W), dtype=np.int64)
    cnt = 0
    for ys in (slice(0, H - ws), slice(H - ws, H - s), slice(H - s, H)):
        for xs in (slice(0, W - ws), slice(W - ws, W - s), slice(W - s, W)):
            region[ys, xs] = cnt
            cnt += 1
    win = rearrange(torch.from_numpy(region), "(a p) (c q) -> (a c) (p q)", p=ws, q=ws).numpy()
    return np.where(win[:, :, None] != win[:, None, :], -100.0, 0.0).astype(np.float32)


def window_token_index_loops(H, W, ws, s):
    """token (row of the natural-order matrix) at position p of window w of the grid rolled by (-s, -s)."""
    out = np.zeros(((H // ws) * (W // ws), ws * ws), dtype=np.int64)
    for wy in range(H // ws):
        for wx in range(W // ws):
            for iy in range(ws):
                for ix in range(ws):
                    out[wy * (W // ws) + wx, iy * ws + ix] = ((wy * ws + iy + s) % H) * W + (wx * ws + ix + s) % W
    return out


def block(sd, x, t_emb):
    p = "modulelist.0."
    m = F.linear(F.silu(F.linear(t_emb, sd[p + "4.modulation.0.weight"], sd[p + "4.modulation.0.bias"])),
                 sd[p + "4.modulation.2.weight"], sd[p + "4.modulation.2.bias"])
    s1, c1, s2, c2 = m.chunk(4, dim=1)
    B, S, d = x.shape
    y = F.layer_norm(x, (d,), sd[p + "0.weight"], sd[p + "0.bias"], 1e-5) * (1 + c1[:, None]) + s1[:, None]
    qkv = F.linear(y, sd[p + "1.to_qkv.weight"], sd[p + "1.to_qkv.bias"])
    g = torch.roll(qkv.reshape(B, H, W, -1), shifts=(-SHIFT, -SHIFT), dims=(1, 2))
    win = rearrange(g, "b (a p) (c q) (t h e) -> t (b a c) h (p q) e", p=WS, q=WS, t=3, h=HEADS)
    idx = torch.from_numpy(relative_position_index_loops(WS))
    bias = sd[p + "1.relative_position_bias_table"][idx.reshape(-1)].reshape(WS * WS, WS * WS, HEADS).permute(2, 0, 1)
    mask = torch.from_numpy(shift_mask_loops(H, W, WS, SHIFT)).repeat(B, 1, 1)
    o = F.scaled_dot_product_attention(win[0], win[1], win[2], attn_mask=bias[None] + mask[:, None])
    o = rearrange(o, "(b a c) h (p q) e -> b (a p) (c q) (h e)", a=H // WS, c=W // WS, p=WS, q=WS)
    o = torch.roll(o, shifts=(SHIFT, SHIFT), dims=(1, 2)).reshape(B, S, -1)
    attn = F.linear(o, sd[p + "1.wo.weight"], sd[p + "1.wo.bias"])
    x1 = x + attn
    z = F.layer_norm(x1, (d,), sd[p + "2.weight"], sd[p + "2.bias"], 1e-5) * (1 + c2[:, None]) + s2[:, None]
    mlp = F.linear(F.gelu(F.linear(z, sd[p + "3.fc1.weight"], sd[p + "3.fc1.bias"])), sd[p + "3.fc2.weight"], sd[p + "3.fc2.bias"])
    return x1 + mlp, attn, mlp


def main():
    torch.manual_seed(0)
    cfg = oracle.OracleConfig.spec(dim=DIM, heads=HEADS, head_dim=HD, mlp_dim=MLP, window_size=(WS, WS), image_shape=(H, W),
                                   mod_ways=2)
    sd = {k: v.double() for k, v in oracle.init_block_weights(cfg, SEED, nontrivial=True).items()}
    g = torch.Generator().manual_seed(SEED + 1)
    x = torch.randn(1, H * W, DIM, generator=g).to(torch.bfloat16).float()  # bf16-representable: the GPU test feeds it as is
    t_emb = torch.randn(1, DIM, generator=g)
    with torch.no_grad():
        out, attn, mlp = block(sd, x.double(), t_emb.double())
    np.savez_compressed(os.path.join(os.path.dirname(os.path.abspath(__file__)), "swin_block_small.npz"),
                        geometry=np.array([H, W, WS, SHIFT, DIM, HEADS, HD, MLP, SEED]), x=x.numpy(), t_emb=t_emb.numpy(),
                        out=out.float().numpy(), attn_branch=attn.float().numpy(), mlp_branch=mlp.float().numpy(),
                        window_token_index=window_token_index_loops(H, W, WS, SHIFT),
                        relative_position_index=relative_position_index_loops(WS),
                        shift_mask=shift_mask_loops(H, W, WS, SHIFT))


if __name__ == "__main__":
    main()
