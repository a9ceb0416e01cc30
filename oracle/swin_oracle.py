"""fp32 CPU restatement of the AERIS Swin denoiser block and model.  TEST INFRASTRUCTURE ONLY.

Functional style: every function takes plain tensors and a ``dict`` of weights keyed like the
reference ``state_dict`` (src/aeris_wp_inference/model.py:386-392 for the per-block layout
``modulelist.{j}.{0..4}``).  All math runs in the dtype of its inputs (fp32 in the tests, fp64
where a test asks for it).  The windowed attention is done the un-fused way - roll the grid,
partition into windows, attend, reverse, roll back - so that it is independent of the folded
address arithmetic the HIP kernels use.

Two presets are covered by one set of switches:

  REF  = what model.py executes: RMSNorm (eps = fp32 machine eps), 6-way adaLN-Zero
         modulation applied BEFORE the norm (model.py:399-401), SwiGLU MLP (model.py:148-159),
         no Linear biases, no relative-position bias, no shift mask.
  SPEC = classic Swin-v1 block the benchmark configurations describe: LayerNorm (eps 1e-5),
         optional scale/shift(/gate) modulation applied AFTER the norm, GELU MLP (exact erf),
         Linear biases, learned relative-position bias table, cyclic-shift attention mask.
"""
from __future__ import annotations

import math
from dataclasses import dataclass, field
from typing import Dict, Optional, Tuple

import numpy as np
import torch
import torch.nn.functional as F

from .index_maps import relative_position_index, shift_attention_mask

_FP32_EPS = float(torch.finfo(torch.float32).eps)  # what torch.nn.RMSNorm(eps=None) uses (model.py:387)


@dataclass
class OracleConfig:
    dim: int
    heads: int
    head_dim: int
    mlp_dim: int
    window_size: Tuple[int, int]
    image_shape: Tuple[int, int]
    norm: str = "layernorm"  # "layernorm" | "rmsnorm"
    mod_order: str = "norm_then_mod"  # "norm_then_mod" | "mod_then_norm"
    mod_ways: int = 0  # 0: no modulation, 2: shift+scale, 3: shift+scale+gate (per branch)
    mlp: str = "gelu"  # "gelu" | "swiglu"
    bias: bool = True
    rel_pos_bias: bool = True
    shift_mask: bool = True
    eps: Optional[float] = None
    # model-level
    n_layers: int = 3  # reference semantics: n_layers - 2 Swin layers (model.py:461)
    sublayers: int = 1
    in_channels: int = 0
    out_channels: int = 0
    max_period: int = 10_000
    use_ape: bool = False

    @property
    def inner(self):
        return self.heads * self.head_dim

    @property
    def norm_eps(self):
        if self.eps is not None:
            return self.eps
        return 1e-5 if self.norm == "layernorm" else _FP32_EPS

    @staticmethod
    def ref(**kw):
        base = dict(norm="rmsnorm", mod_order="mod_then_norm", mod_ways=3, mlp="swiglu",
                    bias=False, rel_pos_bias=False, shift_mask=False)
        base.update(kw)
        return OracleConfig(**base)

    @staticmethod
    def spec(**kw):
        return OracleConfig(**kw)


# --------------------------------------------------------------------------------------
# weights

def _tn(gen, *shape, std=0.02):
    w = torch.empty(*shape, dtype=torch.float32)
    torch.nn.init.trunc_normal_(w, std=std, generator=gen)
    return w


def init_block_weights(cfg: OracleConfig, seed: int = 0, prefix: str = "modulelist.0.",
                       nontrivial: bool = False) -> Dict[str, torch.Tensor]:
    """Seeded random-init weights: trunc-normal(std 0.02) matrices, zero biases, unit norm gains.

    ``nontrivial=True`` perturbs every bias / gain / gate so that a dropped term shows up in a
    comparison (with the plain init the gates are ~0 and the block is ~identity).
    """
    g = torch.Generator().manual_seed(seed)
    d, inner, Hd = cfg.dim, cfg.inner, cfg.mlp_dim
    sd: Dict[str, torch.Tensor] = {}

    def small(*shape):
        return 0.1 * torch.randn(*shape, generator=g) if nontrivial else torch.zeros(*shape)

    def mat(rows, cols):  # nontrivial: unit-gain matrices, so that every branch output is O(1)
        return _tn(g, rows, cols, std=cols ** -0.5 if nontrivial else 0.02)

    for n in ("0", "2"):
        sd[f"{prefix}{n}.weight"] = 1.0 + small(d)
        if cfg.norm == "layernorm":
            sd[f"{prefix}{n}.bias"] = small(d)
    sd[f"{prefix}1.to_qkv.weight"] = mat(3 * inner, d)
    sd[f"{prefix}1.wo.weight"] = mat(d, inner)
    if cfg.bias:
        sd[f"{prefix}1.to_qkv.bias"] = small(3 * inner)
        sd[f"{prefix}1.wo.bias"] = small(d)
    if cfg.rel_pos_bias:
        wy, wx = cfg.window_size
        sd[f"{prefix}1.relative_position_bias_table"] = _tn(g, (2 * wy - 1) * (2 * wx - 1), cfg.heads,
                                                             std=0.5 if nontrivial else 0.02)
    if cfg.mlp == "swiglu":
        sd[f"{prefix}3.w1.weight"] = mat(2 * Hd, d)
        sd[f"{prefix}3.w2.weight"] = mat(d, Hd)
    else:
        sd[f"{prefix}3.fc1.weight"] = mat(Hd, d)
        sd[f"{prefix}3.fc2.weight"] = mat(d, Hd)
        if cfg.bias:
            sd[f"{prefix}3.fc1.bias"] = small(Hd)
            sd[f"{prefix}3.fc2.bias"] = small(d)
    if cfg.mod_ways:
        out = 2 * cfg.mod_ways * d
        sd[f"{prefix}4.modulation.0.weight"] = mat(d, d)
        sd[f"{prefix}4.modulation.0.bias"] = small(d)
        sd[f"{prefix}4.modulation.2.weight"] = mat(out, d)
        b2 = small(out)
        if nontrivial and cfg.mod_ways == 3:
            b2 = b2.clone()
            b2[2 * d:3 * d] += 1.0  # gate_msa ~ 1
            b2[5 * d:6 * d] += 1.0  # gate_mlp ~ 1
        sd[f"{prefix}4.modulation.2.bias"] = b2
    return sd


def init_model_weights(cfg: OracleConfig, seed: int = 0, nontrivial: bool = False) -> Dict[str, torch.Tensor]:
    """Full-model weights keyed like ``LocalAERIS.state_dict()`` (model.py:459-466)."""
    g = torch.Generator().manual_seed(seed + 7919)
    d = cfg.dim
    sd: Dict[str, torch.Tensor] = {}
    sd["input_stage.proj.weight"] = _tn(g, d, cfg.in_channels)
    sd["input_stage.proj.bias"] = 0.1 * torch.randn(d, generator=g) if nontrivial else torch.zeros(d)
    for i in range(cfg.n_layers - 2):
        for j in range(cfg.sublayers):
            sd.update(init_block_weights(cfg, seed=seed * 1000 + i * 10 + j + 1,
                                         prefix=f"layers.{i}.modulelist.{j}.", nontrivial=nontrivial))
    sd["output_stage.norm.weight"] = torch.ones(d) + (0.1 * torch.randn(d, generator=g) if nontrivial else 0)
    if cfg.norm == "layernorm":
        sd["output_stage.norm.bias"] = 0.1 * torch.randn(d, generator=g) if nontrivial else torch.zeros(d)
    sd["output_stage.modulation.0.weight"] = _tn(g, d, d)
    sd["output_stage.modulation.0.bias"] = 0.1 * torch.randn(d, generator=g) if nontrivial else torch.zeros(d)
    sd["output_stage.modulation.2.weight"] = _tn(g, 2 * d, d)
    sd["output_stage.modulation.2.bias"] = 0.1 * torch.randn(2 * d, generator=g) if nontrivial else torch.zeros(2 * d)
    sd["output_stage.head.weight"] = _tn(g, cfg.out_channels, d)
    return sd


# --------------------------------------------------------------------------------------
# pointwise pieces

def layer_norm(x, gamma, beta, eps):
    mu = x.mean(-1, keepdim=True)
    var = ((x - mu) ** 2).mean(-1, keepdim=True)
    y = (x - mu) * torch.rsqrt(var + eps)
    y = y * gamma
    return y + beta if beta is not None else y


def rms_norm(x, gamma, eps):
    """x * rsqrt(mean(x^2) + eps) * w  (torch.nn.RMSNorm, used at model.py:387,389,410)."""
    return x * torch.rsqrt((x * x).mean(-1, keepdim=True) + eps) * gamma


def modulate(x, shift, scale):
    """x * (1 + scale[:, None]) + shift[:, None]; scale None => x + shift  (model.py:121-125)."""
    if scale is None:
        return x + shift.unsqueeze(1)
    return x * (1 + scale.unsqueeze(1)) + shift.unsqueeze(1)


def modulation_mlp(t, w0, b0, w2, b2):
    """Linear -> SiLU -> Linear on the noise-level embedding (model.py:319-325)."""
    h = t @ w0.T + b0
    h = h * torch.sigmoid(h)
    return h @ w2.T + b2


def timestep_embedding(t, dim, max_period=10_000):
    """[sin | cos] sinusoidal embedding (the cos|sin halves are flipped, model.py:127-143)."""
    half = dim // 2
    k = torch.arange(half, dtype=t.dtype)
    freqs = torch.exp(-math.log(max_period) * k / half)
    args = t[:, None] * freqs[None]
    parts = [torch.sin(args), torch.cos(args)]
    if dim % 2:
        # the reference pads one zero after [cos|sin] and then swaps two halves of length
        # (dim)/2 - only even dims are used on the path; keep the simple even-dim layout.
        raise NotImplementedError("odd embedding dims are not on the path")
    return torch.cat(parts, dim=-1)


def positional_encoding_2d(channels, h, w, max_positions=10_000, dtype=torch.float32):
    """Absolute 2-D sin/cos encoding over INPUT channels, ``[h, w, channels]`` (model.py:161-196).

    ch = ceil(C/4)*2; the first ch channels encode the ROW position (``pos_x`` spans h,
    model.py:183), the next ch the column; inside each, sin and cos interleave.
    """
    ch = int(math.ceil(channels / 4) * 2)
    inv_freq = 1.0 / (max_positions ** (torch.arange(0, ch, 2, dtype=torch.float32) / ch))
    rows = torch.arange(h, dtype=torch.float32)[:, None] * inv_freq[None]
    cols = torch.arange(w, dtype=torch.float32)[:, None] * inv_freq[None]
    er = torch.stack((rows.sin(), rows.cos()), dim=-1).flatten(-2)  # [h, ch]
    ec = torch.stack((cols.sin(), cols.cos()), dim=-1).flatten(-2)  # [w, ch]
    emb = torch.cat([er[:, None, :].expand(h, w, ch), ec[None, :, :].expand(h, w, ch)], dim=-1)
    return emb[..., :channels].to(dtype).contiguous()


# --------------------------------------------------------------------------------------
# attention

def window_attention(q, k, v, scale, bias=None, mask=None):
    """softmax((q*scale) k^T + bias + mask) v per (window, head)  (model.py:289-293).

    q, k, v: ``[nW, heads, L, hd]``; bias ``[heads, L, L]``; mask ``[nW, L, L]`` (additive).
    """
    s = (q * scale) @ k.transpose(-1, -2)
    if bias is not None:
        s = s + bias.unsqueeze(0)
    if mask is not None:
        s = s + mask.unsqueeze(1)
    return s.softmax(dim=-1) @ v


def _partition(t, B, H, W, wy, wx):
    # [B, H*W, C] -> [B*nWy*nWx, wy*wx, C]
    C = t.shape[-1]
    t = t.reshape(B, H // wy, wy, W // wx, wx, C).permute(0, 1, 3, 2, 4, 5)
    return t.reshape(B * (H // wy) * (W // wx), wy * wx, C)


def _reverse(t, B, H, W, wy, wx):
    C = t.shape[-1]
    t = t.reshape(B, H // wy, W // wx, wy, wx, C).permute(0, 1, 3, 2, 4, 5)
    return t.reshape(B, H * W, C)


def attention_core(cfg: OracleConfig, qkv, shift, table=None, window_chunk=64):
    """qkv ``[B, S, 3*inner]`` (columns ordered (c h d), model.py:300) -> ``[B, S, inner]``."""
    B, S, _ = qkv.shape
    H, W = cfg.image_shape
    wy, wx = cfg.window_size
    sy, sx = shift
    h, hd, inner = cfg.heads, cfg.head_dim, cfg.inner
    L = wy * wx
    g = qkv.reshape(B, H, W, 3 * inner)
    if sy or sx:
        g = torch.roll(g, shifts=(-sy, -sx), dims=(1, 2))  # model.py:111-112
    win = _partition(g.reshape(B, S, 3 * inner), B, H, W, wy, wx)  # [nW, L, 3*inner]
    nW = win.shape[0]
    win = win.reshape(nW, L, 3, h, hd).permute(2, 0, 3, 1, 4)  # [3, nW, h, L, hd]
    q, k, v = win[0], win[1], win[2]
    bias = None
    if cfg.rel_pos_bias:
        idx = torch.from_numpy(relative_position_index(wy, wx))
        bias = table[idx.reshape(-1)].reshape(L, L, h).permute(2, 0, 1).to(qkv.dtype)
    mask = None
    if cfg.shift_mask and (sy or sx):
        m = torch.from_numpy(shift_attention_mask(H, W, wy, wx, sy, sx)).to(qkv.dtype)
        mask = m.repeat(B, 1, 1)
    out = torch.empty(nW, h, L, hd, dtype=qkv.dtype)
    scale = hd ** -0.5
    for w0 in range(0, nW, window_chunk):  # chunked: the full score tensor is tens of GB at full size
        w1 = min(nW, w0 + window_chunk)
        out[w0:w1] = window_attention(q[w0:w1], k[w0:w1], v[w0:w1], scale, bias,
                                      None if mask is None else mask[w0:w1])
    o = out.permute(0, 2, 1, 3).reshape(nW, L, inner)
    o = _reverse(o, B, H, W, wy, wx).reshape(B, H, W, inner)
    if sy or sx:
        o = torch.roll(o, shifts=(sy, sx), dims=(1, 2))  # model.py:113-114
    return o.reshape(B, S, inner)


def attention_branch(cfg: OracleConfig, sd, prefix, y, shift):
    """to_qkv -> windowed attention -> wo  (model.py:298-309)."""
    qkv = y @ sd[f"{prefix}1.to_qkv.weight"].T
    if cfg.bias:
        qkv = qkv + sd[f"{prefix}1.to_qkv.bias"]
    o = attention_core(cfg, qkv, shift, sd.get(f"{prefix}1.relative_position_bias_table"))
    out = o @ sd[f"{prefix}1.wo.weight"].T
    if cfg.bias:
        out = out + sd[f"{prefix}1.wo.bias"]
    return out


def mlp_branch(cfg: OracleConfig, sd, prefix, z):
    if cfg.mlp == "swiglu":  # model.py:156-159
        gu = z @ sd[f"{prefix}3.w1.weight"].T
        gate, up = gu.chunk(2, dim=-1)
        return (F.silu(gate) * up) @ sd[f"{prefix}3.w2.weight"].T
    h = z @ sd[f"{prefix}3.fc1.weight"].T
    if cfg.bias:
        h = h + sd[f"{prefix}3.fc1.bias"]
    h = 0.5 * h * (1.0 + torch.erf(h / math.sqrt(2.0)))
    out = h @ sd[f"{prefix}3.fc2.weight"].T
    if cfg.bias:
        out = out + sd[f"{prefix}3.fc2.bias"]
    return out


def _norm(cfg, sd, prefix, n, x):
    if cfg.norm == "layernorm":
        return layer_norm(x, sd[f"{prefix}{n}.weight"], sd.get(f"{prefix}{n}.bias"), cfg.norm_eps)
    return rms_norm(x, sd[f"{prefix}{n}.weight"], cfg.norm_eps)


def _norm_mod(cfg, sd, prefix, n, x, shift, scale):
    if shift is None:
        return _norm(cfg, sd, prefix, n, x)
    if cfg.mod_order == "mod_then_norm":  # model.py:400-401
        return _norm(cfg, sd, prefix, n, modulate(x, shift, scale))
    return modulate(_norm(cfg, sd, prefix, n, x), shift, scale)  # model.py:426 order


def block_forward(cfg: OracleConfig, sd, x, t_emb=None, shift=(0, 0), prefix="modulelist.0.",
                  return_branches=False):
    """One Swin block (one sublayer of ``SwinLayer.forward``, model.py:397-401).

    x ``[B, S, d]``; t_emb ``[Bt, d]`` (Bt = 1 or B) or None when ``mod_ways == 0``.
    """
    s1 = c1 = g1 = s2 = c2 = g2 = None
    if cfg.mod_ways:
        m = modulation_mlp(t_emb, sd[f"{prefix}4.modulation.0.weight"], sd[f"{prefix}4.modulation.0.bias"],
                           sd[f"{prefix}4.modulation.2.weight"], sd[f"{prefix}4.modulation.2.bias"])
        parts = m.chunk(2 * cfg.mod_ways, dim=1)
        if cfg.mod_ways == 3:
            s1, c1, g1, s2, c2, g2 = parts  # model.py:399
        else:
            s1, c1, s2, c2 = parts
    a = attention_branch(cfg, sd, prefix, _norm_mod(cfg, sd, prefix, "0", x, s1, c1), shift)
    x1 = x + (g1.unsqueeze(1) * a if g1 is not None else a)
    m_out = mlp_branch(cfg, sd, prefix, _norm_mod(cfg, sd, prefix, "2", x1, s2, c2))
    x2 = x1 + (g2.unsqueeze(1) * m_out if g2 is not None else m_out)
    if return_branches:
        return x2, a, m_out
    return x2


# --------------------------------------------------------------------------------------
# model

def input_stage(cfg: OracleConfig, sd, x, dt, ape=None):
    """(+APE) -> Linear(Cin -> d) ; sinusoidal noise-level embedding  (model.py:346-356)."""
    if ape is not None:
        x = x + ape
    tok = x @ sd["input_stage.proj.weight"].T + sd["input_stage.proj.bias"]
    return tok, timestep_embedding(dt, cfg.dim, cfg.max_period)


def output_stage(cfg: OracleConfig, sd, x, t_emb):
    """norm -> modulate(shift, scale) -> head  (model.py:421-429)."""
    m = modulation_mlp(t_emb, sd["output_stage.modulation.0.weight"], sd["output_stage.modulation.0.bias"],
                       sd["output_stage.modulation.2.weight"], sd["output_stage.modulation.2.bias"])
    shift, scale = m.chunk(2, dim=1)
    if cfg.norm == "layernorm":
        y = layer_norm(x, sd["output_stage.norm.weight"], sd.get("output_stage.norm.bias"), cfg.norm_eps)
    else:
        y = rms_norm(x, sd["output_stage.norm.weight"], cfg.norm_eps)
    return modulate(y, shift, scale) @ sd["output_stage.head.weight"].T


def model_forward(cfg: OracleConfig, sd, x, dt, ape=None, return_hidden=False, block_hook=None):
    """Full denoiser forward (model.py:468-477): odd Swin layers run on the half-window-rolled grid.
    ``block_hook(k, hidden)`` sees the residual stream after the embedding (k = 0) and after block k."""
    tok, t_emb = input_stage(cfg, sd, x, dt, ape)
    wy, wx = cfg.window_size
    k = 0
    if block_hook is not None:
        block_hook(0, tok)
    for i in range(cfg.n_layers - 2):
        shift = (wy // 2, wx // 2) if i % 2 == 1 else (0, 0)
        for j in range(cfg.sublayers):
            tok = block_forward(cfg, sd, tok, t_emb, shift, prefix=f"layers.{i}.modulelist.{j}.")
            k += 1
            if block_hook is not None:
                block_hook(k, tok)
    out = output_stage(cfg, sd, tok, t_emb)
    if return_hidden:
        return out, tok
    return out
