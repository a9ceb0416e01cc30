"""Host-side modules of the AERIS Swin denoiser, same class names / constructor arguments /
state_dict keys as src/aeris_wp_inference/model.py of the reference, running on libaeris_hip.so.

Every module is a parameter container plus an orchestration of the C-ABI kernels
(ops.gemm / ops.window_attention / ops.norm_modulate / ops.modulation_linear ...).
There is no torch arithmetic on the hot path and no CPU fallback.

Two presets of the one parameterised block:
  preset="ref"   what the reference executes (model.py:358-403): RMSNorm, 6-way adaLN-Zero
                 modulation applied before the norm, SwiGLU, no Linear biases, no relative
                 position bias, no shift mask; state_dict keys identical to the reference.
  preset="spec"  classic Swin-v1 block: LayerNorm, modulation (0 / 2 / 3 ways per branch) after
                 the norm, GELU MLP (fc1/fc2), Linear biases, learned relative-position bias
                 table, cyclic-shift attention mask.
"""
from __future__ import annotations

import math
import os
from dataclasses import dataclass
from typing import Optional, Tuple

import torch
import torch.nn as nn

from . import ops

_FP32_EPS = float(torch.finfo(torch.float32).eps)


def _pair(v):
    return (int(v[0]), int(v[1])) if isinstance(v, (tuple, list)) or hasattr(v, "__len__") else (int(v), int(v))


@dataclass
class BlockOptions:
    norm: str = "rmsnorm"  # "layernorm" | "rmsnorm"
    mod_order: str = "mod_then_norm"  # "norm_then_mod" | "mod_then_norm"
    mod_ways: int = 3  # 0 | 2 | 3
    mlp: str = "swiglu"  # "gelu" | "swiglu"
    bias: bool = False
    rel_pos_bias: bool = False
    shift_mask: bool = False
    eps: Optional[float] = None

    @staticmethod
    def make(preset: str = "ref", **overrides) -> "BlockOptions":
        if preset == "ref":
            o = BlockOptions()
        elif preset == "spec":
            o = BlockOptions(norm="layernorm", mod_order="norm_then_mod", mod_ways=0, mlp="gelu", bias=True,
                             rel_pos_bias=True, shift_mask=True)
        else:
            raise ValueError(f"unknown preset {preset!r}")
        for k, v in overrides.items():
            if v is None:
                continue
            if not hasattr(o, k):
                raise TypeError(f"unknown block option {k!r}")
            setattr(o, k, v)
        return o

    @property
    def norm_eps(self):
        if self.eps is not None:
            return self.eps
        return 1e-5 if self.norm == "layernorm" else _FP32_EPS


# ----------------------------------------------------------------------------------------------
# functions of the reference module namespace

def modulate(x, shift, scale):
    """x * (1 + scale[:, None]) + shift[:, None]  (model.py:121-125).  Kept for API parity; the block
    never calls it because the modulation is fused into the norm kernel."""
    if scale is None:
        return x + shift.unsqueeze(1)
    return x * (1 + scale.unsqueeze(1)) + shift.unsqueeze(1)


def timestep_embedding(t: torch.Tensor, dim: int, max_period: int = 10_000):
    """Sinusoidal noise-level embedding [sin | cos], f32 [B, dim]  (model.py:127-143)."""
    return ops.timestep_embedding(t.reshape(-1).float().contiguous(), dim, float(max_period))


def swin_shift(tensor, shift_up, mesh=None, img_shape=None, window_size=None, wp_dims=(1, 1)):
    """Cyclic half-window shift of a [b, H*W, d] token tensor on ONE device (model.py:18-119 with a
    1x1 window-parallel grid, where the halo exchange is a self-exchange and only the roll remains).
    The block never calls this: the shift is folded into the attention kernel's addresses."""
    if tuple(wp_dims) != (1, 1):
        raise NotImplementedError("window parallelism across devices is not part of this build")
    H, W = img_shape
    sy, sx = window_size[0] // 2, window_size[1] // 2
    b, n, d = tensor.shape
    g = tensor.reshape(b, H, W, d)
    g = torch.roll(g, shifts=(-sy, -sx) if shift_up else (sy, sx), dims=(1, 2))
    return g.reshape(b, n, d).contiguous()


# ----------------------------------------------------------------------------------------------
# helper classes

class FeedForward(nn.Module):
    """SwiGLU MLP: w2(silu(gate) * up), [gate | up] = w1(x)  (model.py:148-159)."""

    def __init__(self, dim, hidden_dim):
        super().__init__()
        self.w1 = nn.Linear(dim, 2 * hidden_dim, bias=False)
        self.w2 = nn.Linear(hidden_dim, dim, bias=False)

    def forward(self, x):
        h = ops.gemm(x, self.w1.weight, act="swiglu")
        return ops.gemm(h, self.w2.weight)


class Mlp(nn.Module):
    """GELU MLP: fc2(gelu(fc1(x)))  (classic Swin block; no reference counterpart)."""

    def __init__(self, dim, hidden_dim, bias=True):
        super().__init__()
        self.fc1 = nn.Linear(dim, hidden_dim, bias=bias)
        self.fc2 = nn.Linear(hidden_dim, dim, bias=bias)

    def forward(self, x):
        h = ops.gemm(x, self.fc1.weight, self.fc1.bias, act="gelu")
        return ops.gemm(h, self.fc2.weight, self.fc2.bias)


class PositionalEncoding2D(nn.Module):
    """Absolute 2-D sin/cos encoding over the INPUT channels (model.py:161-196).  Runs once at set-up
    (plain torch); the result is a constant added inside the embedding's A-operand kernel."""

    def __init__(self, channels, max_positions=10_000):
        super().__init__()
        self.channels = int(math.ceil(channels / 4) * 2)
        inv_freq = 1.0 / (max_positions ** (torch.arange(0, self.channels, 2).float() / self.channels))
        self.register_buffer("inv_freq", inv_freq)
        self.register_buffer("cached_penc", None, persistent=False)

    def forward(self, x):
        if x.ndim != 4:
            raise ValueError("input has to be [b, c, h, w]")
        if self.cached_penc is not None and self.cached_penc.shape == x.shape:
            return self.cached_penc
        b, c, h, w = x.shape
        f = self.inv_freq
        rows = torch.arange(h, device=x.device, dtype=f.dtype)[:, None] * f[None]
        cols = torch.arange(w, device=x.device, dtype=f.dtype)[:, None] * f[None]
        er = torch.stack((rows.sin(), rows.cos()), dim=-1).flatten(-2)
        ec = torch.stack((cols.sin(), cols.cos()), dim=-1).flatten(-2)
        emb = torch.cat([er[:, None, :].expand(h, w, -1), ec[None, :, :].expand(h, w, -1)], dim=-1)
        self.cached_penc = emb[..., :c].permute(2, 0, 1)[None].repeat(b, 1, 1, 1).to(x.dtype)
        return self.cached_penc


class RoPE2D(nn.Module):
    """Accepted for constructor parity only: the reference builds it but never applies it
    (the call is commented out at model.py:304) and its buffers are not part of the state_dict."""

    def __init__(self, window_size=None, rope_dim=None, rope_base=10_000):
        super().__init__()
        self.window_size, self.rope_dim, self.rope_base = window_size, rope_dim, rope_base

    def forward(self, x):
        raise NotImplementedError("RoPE2D is not on the executed path of the reference")


# Whether ``Attention`` runs the to_qkv projection inside the attention kernel where that kernel exists (16x16 windows,
# head_dim 64, dim % 128 == 0 and >= 256) instead of as a GEMM that writes q, k, v to HBM for a separate attention
# kernel.  Both paths compute the same bits.  Inside the benchmark's denoiser step the one-kernel form is the faster of
# the two (13.96-13.99 ms against 11.5-11.7 + 2.67-2.68 ms per block, 0.5-0.8 % of the step; bench.py times the step both
# ways in every run), so it is the default; every other shape takes the pair.
FUSE_QKV_ATTENTION = True


class Attention(nn.Module):
    """Windowed multi-head self-attention: to_qkv GEMM -> fused window attention -> wo GEMM
    (model.py:265-309).  ``forward(x, shift=(sy, sx))`` folds a cyclic shift into the kernel."""

    def __init__(self, dim, heads, head_dim, window_size, image_shape, device_mesh=None, wp_dims=(1, 1), *,
                 bias=False, rel_pos_bias=False, shift_mask=False, **rope_kwargs):
        super().__init__()
        if tuple(wp_dims) != (1, 1):
            raise NotImplementedError("window parallelism across devices is not part of this build")
        self.heads, self.head_dim = heads, head_dim
        self.window_size, self.image_shape = _pair(window_size), _pair(image_shape)
        self.scale = head_dim ** -0.5
        self.shift_mask = shift_mask
        self.fuse_qkv = FUSE_QKV_ATTENTION  # per module; see FUSE_QKV_ATTENTION
        self._b4cache = None
        inner = heads * head_dim
        self.rope = RoPE2D(**{k: v for k, v in rope_kwargs.items() if k in ("window_size", "rope_dim", "rope_base")})
        self.to_qkv = nn.Linear(dim, inner * 3, bias=bias)
        self.wo = nn.Linear(inner, dim, bias=bias)
        if rel_pos_bias:
            wy, wx = self.window_size
            self.relative_position_bias_table = nn.Parameter(torch.zeros((2 * wy - 1) * (2 * wx - 1), heads))
            nn.init.trunc_normal_(self.relative_position_bias_table, std=0.02)
        else:
            self.relative_position_bias_table = None

    def _bias4(self):
        """The bias table in the fused kernel's form, refreshed whenever the parameter changes."""
        t = self.relative_position_bias_table
        if t is None:
            return None
        key = (t.data_ptr(), t._version, t.device, t.dtype)
        if self._b4cache is None or self._b4cache[0] != key:
            self._b4cache = (key, ops.qkv_attention_pack_bias(t.detach().to(torch.bfloat16).contiguous(), self.window_size))
        return self._b4cache[1]

    def core(self, y, shift=(0, 0), out=None):
        """y bf16 [b, n, d] -> attention output before ``wo`` (bf16 [b*n, inner])."""
        b, n, _ = y.shape
        use_mask = self.shift_mask and (shift[0] > 0 or shift[1] > 0)
        if self.fuse_qkv and ops.qkv_attention_supported(y.shape[-1], self.heads, self.head_dim, self.window_size,
                                                         self.image_shape):
            # projection and attention in one kernel: q, k, v stay on the chip (same arithmetic, bit-identical result)
            return ops.qkv_window_attention(y.reshape(b * n, -1), self.to_qkv.weight, self.to_qkv.bias, self._bias4(), b,
                                            self.image_shape, self.heads, self.head_dim, self.window_size, shift, use_mask,
                                            self.scale, out=out)
        # q, k, v leave the GEMM as one [b*n, head_dim] plane per part and head (the "(c h d) -> c h d" split of
        # model.py:300 done by the store addresses): a window's rows are then contiguous runs for the attention kernel.
        # The q planes leave the GEMM multiplied by scale * log2(e) in fp32 (model.py:290's `q * self.scale`, in the
        # exp2 domain of the kernel's softmax) so that q is rounded to bf16 once, not twice.
        qkv = ops.gemm_heads(y, self.to_qkv.weight, self.to_qkv.bias, self.head_dim,
                             out=ops.workspace("qkv", (3 * self.heads, b * n, self.head_dim), torch.bfloat16, y.device),
                             q_scale=self.scale * ops.LOG2E, q_planes=self.heads)
        return ops.window_attention(qkv, b, self.image_shape, self.heads, self.head_dim,
                                    self.window_size, shift, self.relative_position_bias_table, use_mask, self.scale, out=out,
                                    head_planes=True, q_prescaled=True)

    def forward(self, x, shift=(0, 0)):
        b, n, d = x.shape
        o = self.core(x, shift)
        return ops.gemm(o, self.wo.weight, self.wo.bias).view(b, n, d)


class ModulationLinear(nn.Module):
    """Linear -> SiLU -> Linear on the noise-level embedding (model.py:311-325); f32 in, f32 out.

    Its parameters stay float32 whatever the enclosing module is cast to (``.to(torch.bfloat16)`` moves them and leaves
    their precision alone).  The shift / scale / gate vectors it produces apply to every token alike, so an error in
    them is not averaged out over tokens or channels: with these 7 d^2 weights per block rounded to bf16 (what the
    reference's bf16 layers hold) the residual stream of a 24-block model with O(1) branch gains is off by 5e-3 from
    this source alone, more than from all four block GEMMs' bf16 weights together.  A bf16 checkpoint loads into them
    without loss; the two matrix-vector products read 66 MB per block and call instead of 33 MB.
    """

    def __init__(self, dim, out_dim, bias):
        super().__init__()
        self.modulation = nn.Sequential(nn.Linear(dim, dim, bias=bias), nn.SiLU(), nn.Linear(dim, out_dim, bias=bias))

    def _apply(self, fn, recurse=True):
        def keep_f32(t):
            r = fn(t)
            if t.dtype == torch.float32 and r.is_floating_point() and r.dtype != torch.float32:
                r = t.to(device=r.device)  # follow a move to another device, not a down-cast
            return r
        return super()._apply(keep_f32, recurse)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        l0, l2 = self.modulation[0], self.modulation[2]
        x = x.float().contiguous()
        h = ops.modulation_linear(x, l0.weight, l0.bias, silu=True)
        return ops.modulation_linear(h, l2.weight, l2.bias)


def _norm_module(opts: BlockOptions, dim):
    if opts.norm == "layernorm":
        return nn.LayerNorm(dim, eps=opts.norm_eps)
    return nn.RMSNorm(dim, eps=opts.eps)


def _norm_call(opts: BlockOptions, norm, x, shift, scale, out=None):
    return ops.norm_modulate(x, norm.weight, getattr(norm, "bias", None), shift, scale, kind=opts.norm,
                             order=opts.mod_order, eps=opts.norm_eps, out=out)


class SwinLayer(nn.Module):
    """``sublayers`` Swin blocks [norm, Attention, norm, MLP, ModulationLinear]  (model.py:358-403).

    forward(x [b, n, d] bf16 | f32, dt [1 | b, d]) -> same shape and dtype as x.
    With preset="ref" the layer, like the reference's, does not shift on its own (the reference
    shifts at model level, model.py:471-475); ``LocalAERIS`` passes ``shift=`` for odd layers.
    With preset="spec" ``shifted_grid=True`` shifts by half a window inside the attention kernel.
    """

    def __init__(self, device_mesh, dim, heads, head_dim, mlp_dim, window_size, image_shape, shifted_grid, rope_base,
                 wp_dims=(1, 1), sublayers=1, *, preset="ref", **options):
        super().__init__()
        self.opts = BlockOptions.make(preset, **options)
        o = self.opts
        self.dim, self.window_size, self.image_shape = dim, _pair(window_size), _pair(image_shape)
        self.sublayers = sublayers
        self.shifted_grid = bool(shifted_grid)
        self.own_shift = preset != "ref"
        rope_kwargs = {"window_size": self.window_size, "rope_dim": head_dim // 2, "rope_base": rope_base}
        blocks = []
        for _ in range(sublayers):
            mods = [
                _norm_module(o, dim),
                Attention(dim, heads, head_dim, image_shape=image_shape, device_mesh=device_mesh, wp_dims=wp_dims,
                          bias=o.bias, rel_pos_bias=o.rel_pos_bias, shift_mask=o.shift_mask, **rope_kwargs),
                _norm_module(o, dim),
                FeedForward(dim, mlp_dim) if o.mlp == "swiglu" else Mlp(dim, mlp_dim, bias=o.bias),
            ]
            if o.mod_ways:
                mods.append(ModulationLinear(dim, 2 * o.mod_ways * dim, bias=True))
            blocks.append(nn.ModuleList(mods))
        self.modulelist = nn.ModuleList(blocks)

    def default_shift(self):
        if self.own_shift and self.shifted_grid:
            return (self.window_size[0] // 2, self.window_size[1] // 2)
        return (0, 0)

    def block_forward(self, j, x, dt, shift, out=None, tap=None):
        """One block.  x is not modified; the result is written to ``out`` (allocated if None).

        ``tap(name, tensor, block)``, if given, is shown the two intermediates the block holds anyway before they are
        consumed: "attn" (attention output ahead of the wo projection) and "hidden" (activated MLP hidden ahead of the
        down projection), both as views of shared scratch that the next kernel overwrites.
        """
        o = self.opts
        mods = self.modulelist[j]
        n1, attn, n2, ff = mods[0], mods[1], mods[2], mods[3]
        b, n, d = x.shape
        s1 = c1 = g1 = s2 = c2 = g2 = None
        if o.mod_ways:
            m = mods[4](dt)  # f32 [1|b, 2*ways*d]
            parts = m.chunk(2 * o.mod_ways, dim=1)
            if o.mod_ways == 3:
                s1, c1, g1, s2, c2, g2 = parts  # model.py:399
            else:
                s1, c1, s2, c2 = parts
        # intermediates live in shared scratch buffers (ops.workspace); only `out` is returned
        y = _norm_call(o, n1, x, s1, c1, out=ops.workspace("norm", (b, n, d), torch.bfloat16, x.device))
        a = attn.core(y, shift, out=ops.workspace("attn", (b * n, attn.wo.weight.shape[1]), torch.bfloat16, x.device))
        if tap is not None:
            tap("attn", a, mods)
        if out is None:
            out = torch.empty_like(x)
        ops.gemm(a, attn.wo.weight, attn.wo.bias, gate=g1, residual=x, rows_per_batch=n, out=out)
        z = _norm_call(o, n2, out, s2, c2, out=y)
        if o.mlp == "swiglu":
            h = ops.gemm(z, ff.w1.weight, act="swiglu",
                         out=ops.workspace("hidden", (b, n, ff.w1.weight.shape[0] // 2), torch.bfloat16, x.device))
            w_dn, b_dn = ff.w2.weight, None
        else:
            h = ops.gemm(z, ff.fc1.weight, ff.fc1.bias, act="gelu",
                         out=ops.workspace("hidden", (b, n, ff.fc1.weight.shape[0]), torch.bfloat16, x.device))
            w_dn, b_dn = ff.fc2.weight, ff.fc2.bias
        if tap is not None:
            tap("hidden", h, mods)
        ops.gemm(h, w_dn, b_dn, gate=g2, residual=out, rows_per_batch=n, out=out)  # in place: out += gate * mlp
        return out

    def forward(self, x, dt=None, shift=None, tap=None):
        if self.opts.mod_ways and dt is None:
            raise ValueError("this layer is modulated: dt (noise-level embedding [1|b, d]) is required")
        shift = self.default_shift() if shift is None else shift
        if x.dtype not in (torch.bfloat16, torch.float32):
            raise TypeError("x must be bf16 or f32")
        x = x.contiguous()
        for j in range(self.sublayers):
            x = self.block_forward(j, x, dt, shift, tap=tap)
        return x


class InputStage(nn.Module):
    """(+APE) -> Linear(Cin -> d) ; sinusoidal noise-level embedding  (model.py:327-356).

    Parameters stay f32 like the reference's, and so does the accuracy of the Linear (fp32 in the reference,
    model.py:352): the input and the weight are each split into a bf16 head and a bf16 remainder and the three
    significant products are summed in fp32 on the matrix cores.  One kernel reads the input channels and the
    positional encoding and writes the token rows (ops.input_stage); shapes it does not take (more than 159 input
    channels, dim not a multiple of 64) go through an operand matrix [x_hi | x_lo | x_hi | 1 | 1] and one bf16 GEMM
    against [W_hi | W_hi | W_lo | b_hi | b_lo].  The split weight is cached and refreshed whenever the parameter
    changes.
    """

    def __init__(self, model_in_channels, dim, sinusoidal_emb_max_period, data_dtype=torch.float32,
                 model_dtype=torch.bfloat16):
        super().__init__()
        self.model_in_channels = model_in_channels
        self.sinusoidal_emb_max_period = sinusoidal_emb_max_period
        self.data_dtype, self.model_dtype = data_dtype, model_dtype
        self.proj = nn.Linear(model_in_channels, dim).to(data_dtype)
        self.ape = PositionalEncoding2D(model_in_channels).to(data_dtype)
        self.ape_generated = None
        self._wcache = None

    def _weights(self, fused):
        w, b = self.proj.weight, self.proj.bias
        key = (w.data_ptr(), w._version, b.data_ptr(), b._version, w.device, fused)
        if self._wcache is None or self._wcache[0] != key:
            c = self.model_in_channels
            w32, b32 = w.detach().float().contiguous(), b.detach().float().contiguous()
            if fused:
                self._wcache = (key, ops.input_stage_pack_weight(w32, b32), 0)
            else:
                k_pad = (3 * c + 2 + 63) // 64 * 64
                w_hi, b_hi = w32.to(torch.bfloat16), b32.to(torch.bfloat16)
                w_lo, b_lo = (w32 - w_hi.float()).to(torch.bfloat16), (b32 - b_hi.float()).to(torch.bfloat16)
                wp = torch.zeros(w.shape[0], k_pad, dtype=torch.bfloat16, device=w.device)
                wp[:, :c], wp[:, c:2 * c], wp[:, 2 * c:3 * c] = w_hi, w_hi, w_lo
                wp[:, 3 * c], wp[:, 3 * c + 1] = b_hi, b_lo
                self._wcache = (key, wp, k_pad)
        return self._wcache[1:]

    def forward(self, x, interval, out_dtype=None, cond=None, x_div=1.0):
        """x [b, n, Cin]; or x [b, n, C0] with cond [b, n, Cin - C0]: the embedding of cat([x / x_div, cond], 2)
        (inference.py:160) without building the concatenated tensor."""
        b, n, c = x.shape
        if cond is not None:
            c += cond.shape[-1]
        if c != self.model_in_channels:
            raise ValueError(f"input has {c} channels, the model embeds {self.model_in_channels}")
        ape = self.ape_generated
        if ape is not None:
            ape = ape.reshape(-1, c)
            if ape.shape[0] != n:
                raise ValueError(f"ape_generated covers {ape.shape[0]} tokens, input has {n}")
        dim = self.proj.weight.shape[0]
        fused = ops.input_stage_supported(c, dim) and (ape is None or ape.shape[0] >= 64)
        wp, k_pad = self._weights(fused)
        x2 = x.reshape(b * n, -1).float().contiguous()
        c2 = None if cond is None else cond.reshape(b * n, -1).float().contiguous()
        if fused:
            tok = ops.input_stage(x2, x_div if cond is not None else 1.0, c2, ape, wp, dim,
                                  out_dtype=out_dtype or self.model_dtype).view(b, n, -1)
        else:
            if cond is None:
                a = ops.embed_prepare(x2, ape, k_pad, split=True)
            else:
                a = ops.embed_concat(x2, x_div, c2, ape, k_pad, split=True)
            tok = ops.gemm(a, wp, None, out_dtype=out_dtype or self.model_dtype).view(b, n, -1)
        t = timestep_embedding(interval, tok.shape[-1], self.sinusoidal_emb_max_period)
        return tok, t


class OutputStage(nn.Module):
    """norm -> modulate(shift, scale) -> head  (model.py:405-429); f32 parameters, f32 arithmetic accuracy and f32
    output like the reference's.  One fused kernel reads the tokens once (ops.output_stage); shapes it does not take
    (more than 80 output channels, dim not a multiple of 64) run as norm kernel + bf16 GEMM."""

    def __init__(self, dim, model_out_channels, image_shape, data_dtype=torch.float32, *, norm="rmsnorm", eps=None):
        super().__init__()
        self.data_dtype, self.image_shape = data_dtype, image_shape
        self.norm_kind = norm
        self.norm_eps = eps if eps is not None else (1e-5 if norm == "layernorm" else _FP32_EPS)
        self.norm = (nn.LayerNorm(dim, eps=self.norm_eps) if norm == "layernorm" else nn.RMSNorm(dim)).to(data_dtype)
        self.modulation = nn.Sequential(nn.Linear(dim, dim, bias=True), nn.SiLU(), nn.Linear(dim, 2 * dim, bias=True))
        self.head = nn.Linear(dim, model_out_channels, bias=False).to(data_dtype)
        self._wcache = None

    def _head_weight(self):
        w = self.head.weight
        key = (w.data_ptr(), w._version, w.device)
        if self._wcache is None or self._wcache[0] != key:
            self._wcache = (key, w.detach().to(torch.bfloat16).contiguous())
        return self._wcache[1]

    def forward(self, x, dt):
        b, n, d = x.shape
        l0, l2 = self.modulation[0], self.modulation[2]
        h = ops.modulation_linear(dt.float().contiguous(), l0.weight, l0.bias, silu=True)
        m = ops.modulation_linear(h, l2.weight, l2.bias)
        shift, scale = m.chunk(2, dim=1)  # model.py:425
        beta = getattr(self.norm, "bias", None)
        w = self.head.weight
        if w.dtype == torch.float32 and ops.output_stage_supported(w.shape[0], d, m.shape[0] if b > 1 else 1, n):
            return ops.output_stage(x.contiguous(), self.norm.weight, beta, shift, scale, w, kind=self.norm_kind,
                                    eps=self.norm_eps)
        y = ops.norm_modulate(x.contiguous(), self.norm.weight, beta, shift, scale, kind=self.norm_kind,
                              order="norm_then_mod", eps=self.norm_eps)
        return ops.gemm(y, self._head_weight(), out_dtype=torch.float32).view(b, n, -1)


class LocalAERIS(nn.Module):
    """The denoiser: InputStage -> (n_layers - 2) SwinLayers, odd ones on the half-window-shifted grid
    -> OutputStage  (model.py:431-477).  forward(x [B, S, Cin] f32, dt [1] f32) -> [B, S, Cout] f32.

    ``residual_dtype`` selects the dtype of the residual stream between blocks: f32 (default), or bf16 like the
    reference's bf16 layers.  With a bf16 stream the two roundings per block add up to more than 1e-2 of the stream
    after 24 blocks; with f32 the result stays within 1e-2 of an fp32 evaluation at that depth.
    """

    def __init__(self, device_mesh=None, heads=None, dim=None, head_dim=None, mlp_dim=None, window_size=None,
                 image_shape=None, rope_base=10_000, sublayers=1, sinusoidal_emb_max_period=10_000, n_layers=None,
                 model_in_channels=None, model_out_channels=None, SP=1, sp_rank=1, wp_dims=(1, 1), *, preset="ref",
                 residual_dtype=torch.float32, **options):
        super().__init__()
        if tuple(wp_dims) != (1, 1) or SP != 1:
            raise NotImplementedError("this build runs the whole grid on one device (SP = 1, wp_dims = (1, 1))")
        model_dtype, data_dtype = torch.bfloat16, torch.float32
        self.mesh = device_mesh
        self.image_shape, self.window_size = _pair(image_shape), _pair(window_size)
        self.wp_dims, self.heads = wp_dims, heads
        self.residual_dtype = residual_dtype
        self.opts = BlockOptions.make(preset, **options)
        self.input_stage = InputStage(model_in_channels, dim, sinusoidal_emb_max_period).to(data_dtype)
        layers = []
        for i in range(n_layers - 2):
            layers.append(SwinLayer(device_mesh, dim, heads, head_dim, mlp_dim, window_size, image_shape, i % 2 == 1,
                                    rope_base, sublayers=sublayers, wp_dims=wp_dims, preset=preset, **options))
        self.layers = nn.ModuleList(layers).to(model_dtype)
        self.output_stage = OutputStage(dim, model_out_channels, image_shape, norm=self.opts.norm,
                                        eps=self.opts.eps).to(data_dtype)

    def generate_ape(self, device=None):
        """APE as inference.py:283 builds it: encode an (H+1)-row grid, drop row 0, flatten row-major."""
        H, W = self.image_shape
        c = self.input_stage.model_in_channels
        device = device or self.input_stage.proj.weight.device
        pe = self.input_stage.ape(torch.zeros((1, c, H + 1, W), dtype=torch.float32, device=device))[:, :, 1:, :]
        self.input_stage.ape_generated = pe.permute(0, 2, 3, 1).reshape(1, H * W, c).contiguous()
        return self.input_stage.ape_generated

    def forward(self, x, dt, return_hidden=False, cond=None, x_div=1.0, block_hook=None):
        """``cond`` / ``x_div``: see InputStage.forward (the sampler's concatenation folded into the embedding).
        ``block_hook(k, hidden)`` is called with the residual stream after the embedding (k = 0) and after every
        block (k = 1..); the tensor is reused by later blocks, so a hook that keeps it must copy it."""
        tok, t = self.input_stage(x, dt, out_dtype=self.residual_dtype, cond=cond, x_div=x_div)
        if block_hook is not None:
            block_hook(0, tok)
        k = 0
        half = (self.window_size[0] // 2, self.window_size[1] // 2)
        spare = None
        for i, layer in enumerate(self.layers):
            shift = half if i % 2 == 1 else (0, 0)  # model.py:471-475, folded into the attention kernel
            for j in range(layer.sublayers):
                if spare is None:
                    spare = torch.empty_like(tok)
                res = layer.block_forward(j, tok, t, shift, out=spare)
                tok, spare = res, tok
                k += 1
                if block_hook is not None:
                    block_hook(k, tok)
        out = self.output_stage(tok, t)
        return (out, tok) if return_hidden else out


def convert_inference_checkpoint(path, N, model, map_location="cpu"):
    """Stitch the per-pipeline-stage ``ema_state_dict`` files of a training run into ``model``
    (model.py:479-495): stage 0 -> input_stage.*, stage k -> layers.{k-1}.*, stage N-1 ->
    output_stage.*; stray ``latent_embed`` / ``1.norm`` entries are dropped."""
    def load(k):
        f = os.path.join(path, f"checkpoint_PP{k}.pth")
        return torch.load(f, map_location=map_location, weights_only=True)["ema_state_dict"]

    merged = {}
    for key, v in load(0).items():
        if "latent_embed" not in key:
            merged[f"input_stage.{key}"] = v
    for i in range(N - 2):
        for key, v in load(i + 1).items():
            if "1.norm" not in key:
                merged[f"layers.{i}.{key}"] = v
    for key, v in load(N - 1).items():
        merged[f"output_stage.{key}"] = v
    want = set(model.state_dict().keys())
    if want != set(merged.keys()):
        missing, extra = sorted(want - set(merged)), sorted(set(merged) - want)
        raise KeyError(f"checkpoint does not match the model 1:1; missing {missing[:5]}, unexpected {extra[:5]}")
    model.load_state_dict(merged)
