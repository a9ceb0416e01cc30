"""Writes tests/golden/ref_block_small.npz: inputs and expected outputs of the reference's own block form
(src/aeris_wp_inference/model.py: RMSNorm with eps=None, six-way modulation applied BEFORE the norm, SwiGLU, no biases,
no relative-position bias, no mask; the cyclic half-window shift applied to the residual stream around the layer), once
un-shifted and once between the two shifts.

The reference ships no tests or vectors and was not run.  The expected values are composed, in float64, from library
routines called the way model.py calls them - torch.nn.RMSNorm (model.py:387,389), einops.rearrange with the
pattern strings of model.py:300,302,307, F.scaled_dot_product_attention (the reference's own alternative to its naive
attention, model.py:295-296, same scale), F.silu, F.linear, torch.roll (model.py:111-114) - and NOT with any function of
oracle/: the fixture pins the oracle's op order (modulate -> norm -> branch -> gate -> residual, model.py:399-401) from the
outside.  Only the seeded weights come from oracle.init_block_weights (data, not arithmetic).

    python tests/golden/make_golden_ref.py        # rewrites the .npz next to this file
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

H, W, WS_Y, WS_X = 24, 24, 12, 8       # rectangular windows; head_dim 128 is the streaming attention kernel's territory
DIM, HEADS, HD, MLP = 128, 2, 128, 192
SEED = 11


def layer(sd, x, t_emb):
    """SwinLayer.forward with one sublayer (model.py:395-403), Attention.forward (model.py:298-309), FeedForward (model.py:156-159)."""
    p = "modulelist.0."
    d = x.shape[-1]
    n1, n2 = torch.nn.RMSNorm(d).double(), torch.nn.RMSNorm(d).double()
    n1.weight.data.copy_(sd[p + "0.weight"])
    n2.weight.data.copy_(sd[p + "2.weight"])
    mod = F.linear(F.silu(F.linear(t_emb, sd[p + "4.modulation.0.weight"], sd[p + "4.modulation.0.bias"])),
                   sd[p + "4.modulation.2.weight"], sd[p + "4.modulation.2.bias"])
    shift_msa, scale_msa, gate_msa, shift_mlp, scale_mlp, gate_mlp = mod.chunk(6, dim=1)

    y = n1(x * (1 + scale_msa.unsqueeze(1)) + shift_msa.unsqueeze(1))
    qkv = F.linear(y, sd[p + "1.to_qkv.weight"])
    qkv = rearrange(qkv, "b n (c h d) -> b n h (c d)", c=3, h=HEADS)
    qkv = rearrange(qkv, "b (wcl_y ws_y wcl_x ws_x) h d -> (b wcl_y wcl_x) h (ws_y ws_x) d", wcl_y=H // WS_Y, wcl_x=W // WS_X,
                    ws_y=WS_Y, ws_x=WS_X)
    q, k, v = qkv.chunk(3, dim=-1)
    o = F.scaled_dot_product_attention(q, k, v, is_causal=False)
    o = rearrange(o, "(b wcl_y wcl_x) h (ws_y ws_x) d -> b (wcl_y ws_y wcl_x ws_x) (h d)", wcl_y=H // WS_Y, wcl_x=W // WS_X,
                  ws_y=WS_Y, ws_x=WS_X)
    attn = F.linear(o, sd[p + "1.wo.weight"])
    x = x + gate_msa.unsqueeze(1) * attn

    z = n2(x * (1 + scale_mlp.unsqueeze(1)) + shift_mlp.unsqueeze(1))
    gate, up = F.linear(z, sd[p + "3.w1.weight"]).chunk(2, dim=-1)
    ff = F.linear(F.silu(gate) * up, sd[p + "3.w2.weight"])
    return x + gate_mlp.unsqueeze(1) * ff


def roll_tokens(x, up):
    """swin_shift on one device (model.py:37,111-116): the token grid rolled by half a window, up or back down."""
    B = x.shape[0]
    g = x.reshape(B, H, W, -1)
    sh = (-(WS_Y // 2), -(WS_X // 2)) if up else (WS_Y // 2, WS_X // 2)
    return torch.roll(g, shifts=sh, dims=(1, 2)).reshape(B, H * W, -1)


def main():
    torch.manual_seed(0)
    cfg = oracle.OracleConfig.ref(dim=DIM, heads=HEADS, head_dim=HD, mlp_dim=MLP, window_size=(WS_Y, WS_X), image_shape=(H, W))
    sd = {k: v.double() for k, v in oracle.init_block_weights(cfg, SEED, nontrivial=True).items()}
    g = torch.Generator().manual_seed(SEED + 1)
    x = torch.randn(1, H * W, DIM, generator=g).to(torch.bfloat16).float()  # bf16-representable: the GPU test feeds it as is
    t_emb = torch.randn(1, DIM, generator=g)
    with torch.no_grad():
        plain = layer(sd, x.double(), t_emb.double())
        shifted = roll_tokens(layer(sd, roll_tokens(x.double(), True), t_emb.double()), False)
    np.savez_compressed(os.path.join(os.path.dirname(os.path.abspath(__file__)), "ref_block_small.npz"),
                        geometry=np.array([H, W, WS_Y, WS_X, DIM, HEADS, HD, MLP, SEED]), x=x.numpy(), t_emb=t_emb.numpy(),
                        out_plain=plain.float().numpy(), out_shifted=shifted.float().numpy())


if __name__ == "__main__":
    main()
