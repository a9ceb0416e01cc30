"""GPU parity tests of each HIP kernel, called through the C ABI, against the CPU oracle.

Tolerances: index maps bit-exact; bf16 results within relative L2 <= 1e-2 of the fp32 oracle
(most kernels are far tighter, each bound is written at its assert).
"""
import math

import numpy as np
import pytest
import torch

import oracle
from oracle import OracleConfig
from oracle.swin_oracle import attention_core

pytestmark = pytest.mark.gpu


def rel_l2(a, b):
    a, b = a.double().cpu(), b.double().cpu()
    return float((a - b).norm() / b.norm().clamp_min(1e-30))


def bf(t):
    return t.to(torch.bfloat16)


# ---------------------------------------------------------------------------------------------- GEMM

GEMM_CASES = [
    # M, N, K, act, bias, gate(batch), residual dtype, out dtype
    (256, 256, 64, None, False, 0, None, torch.bfloat16),
    (1000, 384, 128, None, True, 0, None, torch.bfloat16),        # ragged M, N = 3*128
    (2048, 512, 128, "gelu", True, 0, None, torch.bfloat16),      # configs[0] fc1
    (2048, 128, 512, None, True, 1, torch.bfloat16, torch.bfloat16),  # configs[0] fc2 + gate + residual
    (777, 128, 192, "silu", False, 0, None, torch.float32),
    (4096, 69, 256, None, False, 0, None, torch.float32),         # head: N = 69, scalar epilogue
    (1300, 200, 64, None, True, 0, torch.float32, torch.float32),  # N % 128 != 0, vector epilogue
    (66000, 1536, 512, None, True, 0, None, torch.bfloat16),      # big tiles (256x256), ragged M
    (65536, 512, 2048, None, True, 4, torch.float32, torch.float32),  # big tiles, per-batch gate, f32 residual stream
    (66000, 2048, 512, "gelu", True, 0, None, torch.bfloat16),
    (3000, 256, 128, "swiglu", False, 0, None, torch.bfloat16),   # small-tile SwiGLU
    (70000, 1024, 256, "swiglu", True, 0, None, torch.bfloat16),  # big-tile SwiGLU
    (500, 100, 64, "swiglu", False, 0, None, torch.float32),      # SwiGLU with ragged N
    # big tiles whose rows straddle a batch boundary (64 800 rows per batch = 253 tiles + 32 rows): per-lane gate rows
    (129600, 768, 256, None, True, 2, torch.bfloat16, torch.bfloat16),
    (129600, 512, 128, None, False, 2, torch.float32, torch.float32),
    # 100 rows per batch: every 128-row group of a big tile straddles one or two batch boundaries
    (64000, 512, 128, None, True, 640, torch.bfloat16, torch.bfloat16),
    (64000, 256, 64, None, True, 640, torch.float32, torch.float32),
    (66000, 1028, 64, None, True, 0, torch.bfloat16, torch.bfloat16),  # big tiles, one k-tile, last 16-byte chunk half inside
    (70000, 1100, 128, "swiglu", True, 0, None, torch.bfloat16),  # big-tile SwiGLU with ragged N
    (300, 4096, 192, "gelu", True, 0, torch.bfloat16, torch.bfloat16),  # 2 x 16 big tiles: most workgroups idle or one tile
]


@pytest.mark.parametrize("case", GEMM_CASES, ids=lambda c: f"M{c[0]}_N{c[1]}_K{c[2]}_{c[3]}")
def test_gemm_parity(pkg, cuda, case):
    M, N, K, act, has_bias, gate_b, res_dt, out_dt = case
    g = torch.Generator().manual_seed(M + N + K)
    a = bf(torch.randn(M, K, generator=g))
    n_w = 2 * N if act == "swiglu" else N
    w = bf(torch.randn(n_w, K, generator=g) / math.sqrt(K))
    bias = bf(0.5 * torch.randn(n_w, generator=g)) if has_bias else None
    gate = torch.randn(gate_b, N, generator=g) if gate_b else None
    res = torch.randn(M, N, generator=g).to(res_dt) if res_dt is not None else None
    # fp32 reference on the same (bf16-rounded) operands
    ref = a.float() @ w.float().T
    if bias is not None:
        ref = ref + bias.float()
    if act == "gelu":
        ref = torch.nn.functional.gelu(ref)
    elif act == "silu":
        ref = torch.nn.functional.silu(ref)
    elif act == "swiglu":
        ref = torch.nn.functional.silu(ref[:, :N]) * ref[:, N:]
    if gate is not None:
        rpb = M // gate_b
        ref = ref * gate.repeat_interleave(rpb, dim=0)
    if res is not None:
        ref = ref + res.float()
    dev = lambda t: None if t is None else t.to(cuda)
    out = pkg.ops.gemm(dev(a), dev(w), dev(bias), act=act, gate=dev(gate), residual=dev(res),
                       rows_per_batch=(M // gate_b if gate_b else 0), out_dtype=out_dt)
    torch.cuda.synchronize()
    assert out.shape == (M, N) and out.dtype == out_dt
    err = rel_l2(out, ref)
    assert err <= (3e-3 if out_dt == torch.bfloat16 else 2e-5), err
    assert torch.isfinite(out).all()


def test_gemm_gelu_epilogue_pointwise(pkg, cuda):
    """The GELU of the GEMM epilogue, value by value: with one non-zero column in A and ones in W every output is
    GELU(x) for a chosen x.  Against the erf form in float64: the epilogue's polynomial is within 2.1e-4 |x| (a tenth of
    half a bf16 ulp; above 3.5 this is the clamp's 1 - Phi(3.5)) before the result is rounded to bf16; below -3.5,
    however far, it is the constant -8.1e-4 (the exact value lies between that and 0)."""
    M, N, K = 8192, 256, 64
    x = bf(torch.cat([torch.linspace(-8, 8, M - 2048 - 512), torch.linspace(-0.05, 0.05, 2048),
                      -torch.logspace(math.log10(3.5), 4, 256), torch.logspace(math.log10(3.5), 4, 256)]))
    a = torch.zeros(M, K, dtype=torch.bfloat16)
    a[:, 0] = x
    w = torch.zeros(N, K, dtype=torch.bfloat16)
    w[:, 0] = 1.0
    out = pkg.ops.gemm(a.to(cuda), w.to(cuda), None, act="gelu").float().cpu()
    xd = x.double()
    exact = 0.5 * xd * (1.0 + torch.erf(xd / math.sqrt(2.0)))
    bound = torch.where(xd >= -3.5, 2.1e-4 * xd.abs(), torch.full_like(xd, 8.2e-4)) + 2.0 ** -8 * exact.abs() + 1e-30
    err = (out.double() - exact[:, None]).abs()
    assert bool((err <= bound[:, None]).all()), float((err / bound[:, None]).max())
    assert torch.equal(out, out[:, :1].expand_as(out))  # every column took the same path
    # where the values are not small against |x| (x >= -1): within one bf16 ulp of the exact value
    core = xd >= -1
    assert bool((err[core] <= 2.0 ** -7 * exact[core].abs()[:, None] + 1e-30).all())


def test_gemm_residual_in_place_and_deterministic(pkg, cuda):
    g = torch.Generator().manual_seed(0)
    a, w = bf(torch.randn(5000, 256, generator=g)).to(cuda), bf(torch.randn(384, 256, generator=g) / 16).to(cuda)
    x = torch.randn(5000, 384, generator=g).to(cuda)
    want = pkg.ops.gemm(a, w, residual=x, out_dtype=torch.float32)
    y = x.clone()
    pkg.ops.gemm(a, w, residual=y, out=y)  # C aliases the residual
    assert torch.equal(y, want)
    assert torch.equal(pkg.ops.gemm(a, w, residual=x, out_dtype=torch.float32), want)


# ---------------------------------------------------------------------------------------------- attention

ATTN_CASES = [
    # B, H, W, heads, hd, ws, shift, bias, mask
    (1, 32, 64, 4, 32, 8, 0, False, False),
    (1, 32, 64, 4, 32, 8, 4, True, True),       # configs[0] geometry
    (2, 16, 24, 2, 64, 8, 4, True, True),
    (1, 36, 48, 8, 64, 12, 6, True, True),      # configs[1] window (L = 144, padded to 160)
    (2, 24, 24, 3, 32, 12, 6, True, False),
    (1, 48, 64, 3, 64, 16, 8, True, True),      # configs[2]/[3] window (L = 256)
    (2, 32, 32, 2, 64, 16, 0, False, False),
    (1, 32, 48, 2, 32, 16, 8, False, True),
    (1, 16, 16, 1, 64, 16, 8, True, True),      # one window: every border region in it
    # more (window, head) units than the chip runs at once (2 workgroups per CU), many heads, an odd head count
    (1, 160, 160, 24, 64, 16, 8, True, True),   # configs[3] heads: 2400 units
    (2, 16, 192, 90, 64, 16, 8, True, True),    # 2160 units, 90 heads
    (1, 64, 96, 90, 64, 16, 0, False, False),   # 2160 units, no bias
    (1, 48, 720, 17, 64, 16, 8, True, False),   # 2295 units, 17 heads
]


@pytest.mark.parametrize("case", ATTN_CASES, ids=lambda c: f"B{c[0]}_{c[1]}x{c[2]}_h{c[3]}x{c[4]}_ws{c[5]}_s{c[6]}_b{int(c[7])}m{int(c[8])}")
def test_window_attention_parity(pkg, cuda, case):
    B, H, W, heads, hd, ws, sh, has_bias, use_mask = case
    g = torch.Generator().manual_seed(H * W + heads)
    inner = heads * hd
    qkv = bf(torch.randn(B, H * W, 3 * inner, generator=g))
    table = bf(0.7 * torch.randn((2 * ws - 1) ** 2, heads, generator=g)) if has_bias else None
    cfg = OracleConfig(dim=inner, heads=heads, head_dim=hd, mlp_dim=inner, window_size=(ws, ws), image_shape=(H, W),
                       rel_pos_bias=has_bias, shift_mask=use_mask)
    ref = attention_core(cfg, qkv.float(), (sh, sh), None if table is None else table.float())
    out = pkg.ops.window_attention(qkv.to(cuda).view(B * H * W, -1), B, (H, W), heads, hd, (ws, ws), (sh, sh),
                                   None if table is None else table.to(cuda), use_mask)
    torch.cuda.synchronize()
    err = rel_l2(out.view(B, H * W, inner), ref)
    assert err <= 6e-3, err  # P and O are rounded to bf16 once each
    assert (out.float().cpu().view(B, H * W, inner) - ref).abs().max() < 0.06


PLANE_CASES = [
    # B, H, W, heads, hd, ws, shift, bias, mask, magnitude of q and k -- q / k / v as head planes: the kernels that bring
    # K and V into LDS with buffer_load ... lds and read V^T with the transposing LDS read
    (1, 160, 160, 24, 64, 16, 8, True, True, 1.0),    # persistent form (2400 units), configs[3] heads
    (2, 96, 96, 8, 64, 12, 6, True, True, 1.0),       # persistent form, L = 144 padded to 160 (1024 units)
    (2, 128, 128, 2, 64, 8, 4, True, True, 1.0),      # persistent form, 8x8 windows, two waves per workgroup
    (1, 160, 160, 24, 64, 16, 0, False, False, 1.0),  # persistent form without bias: accumulators start at a literal zero
    (3, 32, 48, 2, 64, 16, 8, True, True, 1.0),       # one workgroup per unit (36 units)
    (1, 36, 48, 3, 64, 12, 6, False, True, 1.0),
    # logits far outside the range in which exp2 can do without the row maximum: rows take the two-pass form
    (1, 160, 160, 24, 64, 16, 8, True, True, 6.0),
    (1, 32, 48, 2, 64, 16, 8, False, False, 8.0),
    (1, 32, 64, 4, 32, 8, 4, True, True, 8.0),        # head_dim 32: the register-staged kernel, same range check
]


LOG2E = 1.4426950408889634


@pytest.mark.parametrize("prescaled", [True, False], ids=["qscaled", "qraw"])
@pytest.mark.parametrize("case", PLANE_CASES, ids=lambda c: f"B{c[0]}_{c[1]}x{c[2]}_h{c[3]}x{c[4]}_ws{c[5]}_s{c[6]}_b{int(c[7])}m{int(c[8])}_x{c[9]:g}")
def test_window_attention_planes_parity(pkg, cuda, case, prescaled):
    """``prescaled``: the q planes hold bf16(q * scale * log2 e), the form the to_qkv GEMM of the model writes (the
    factor applied in fp32 before q's only rounding); the oracle is given exactly those queries (divided by the factor
    again, in fp32), so what is compared is the kernel's own arithmetic: P and O rounded to bf16 once each, at any
    logit magnitude.  Not prescaled: the kernel multiplies the bf16 q by the factor and rounds again (as the
    reference's bf16 `q * self.scale` does, model.py:290), which moves a logit by 2^-9 of its magnitude: nothing at
    ordinary magnitudes, a few percent of P once logits reach the hundreds."""
    B, H, W, heads, hd, ws, sh, has_bias, use_mask, mag = case
    g = torch.Generator().manual_seed(H * W + heads + int(mag))
    inner, S = heads * hd, B * H * W
    qkv = torch.randn(B, H * W, 3 * inner, generator=g)
    qkv[..., :2 * inner] *= mag  # logits of magnitude mag^2 * sqrt(hd) * scale: up to several hundred, and as far below zero
    c = hd ** -0.5 * LOG2E
    if prescaled:
        q_dev = bf(qkv[..., :inner] * c)
        kv = bf(qkv[..., inner:])
        dev_in = torch.cat([q_dev, kv], dim=-1)
        ref_in = torch.cat([q_dev.float() / c, kv.float()], dim=-1)
    else:
        dev_in = bf(qkv)
        ref_in = dev_in.float()
    table = bf(0.7 * torch.randn((2 * ws - 1) ** 2, heads, generator=g)) if has_bias else None
    cfg = OracleConfig(dim=inner, heads=heads, head_dim=hd, mlp_dim=inner, window_size=(ws, ws), image_shape=(H, W),
                       rel_pos_bias=has_bias, shift_mask=use_mask)
    ref = attention_core(cfg, ref_in, (sh, sh), None if table is None else table.float())
    planes = dev_in.view(S, 3 * heads, hd).permute(1, 0, 2).contiguous().to(cuda)  # plane c * heads + h = part c of head h
    out = pkg.ops.window_attention(planes, B, (H, W), heads, hd, (ws, ws), (sh, sh), None if table is None else table.to(cuda),
                                   use_mask, head_planes=True, q_prescaled=prescaled)
    out2 = pkg.ops.window_attention(planes, B, (H, W), heads, hd, (ws, ws), (sh, sh), None if table is None else table.to(cuda),
                                    use_mask, head_planes=True, q_prescaled=prescaled)
    torch.cuda.synchronize()
    assert torch.equal(out, out2)
    assert bool(torch.isfinite(out.float()).all())
    err = rel_l2(out.view(B, H * W, inner), ref)
    print(f"planes attention, |q|,|k| x{mag}, prescaled {prescaled}: rel-L2 {err:.3e}")
    assert err <= (6e-3 if (mag == 1.0 or prescaled) else 3e-2), err
    if mag == 1.0:
        assert (out.float().cpu().view(B, H * W, inner) - ref).abs().max() < 0.06


STREAM_CASES = [
    # B, H, W, heads, head_dim, ws_y, ws_x, shift_y, shift_x  -- shapes only the streaming kernel takes
    (1, 120, 120, 2, 128, 60, 60, 30, 30),   # the reference's window: 3600 tokens, head_dim 128 (model.py:22-27), shifted
    (1, 60, 120, 1, 128, 60, 60, 0, 0),
    (2, 40, 60, 3, 64, 20, 20, 10, 10),      # L = 400: partial last key chunk and query block
    (1, 32, 32, 2, 128, 16, 16, 8, 8),       # L = 256 with head_dim 128
    (1, 24, 40, 2, 128, 12, 20, 6, 10),      # rectangular window, L = 240
    (1, 18, 14, 1, 64, 9, 7, 4, 3),          # L = 63: less than one key chunk, odd sizes
    (1, 64, 128, 2, 64, 64, 64, 32, 32),     # L = 4096, the largest window
]


@pytest.mark.parametrize("case", STREAM_CASES, ids=lambda c: f"B{c[0]}_{c[1]}x{c[2]}_h{c[3]}x{c[4]}_ws{c[5]}x{c[6]}_s{c[7]}x{c[8]}")
def test_window_attention_streaming_parity(pkg, cuda, case):
    """Windows of more than 256 tokens and head_dim 128 (no bias, no mask: what the reference's model.py runs) go
    through the streaming kernel; same oracle, same tolerance as the one-window-per-workgroup kernel."""
    B, H, W, heads, hd, wsy, wsx, shy, shx = case
    g = torch.Generator().manual_seed(H * W + heads)
    inner = heads * hd
    qkv = bf(torch.randn(B, H * W, 3 * inner, generator=g))
    cfg = OracleConfig(dim=inner, heads=heads, head_dim=hd, mlp_dim=inner, window_size=(wsy, wsx), image_shape=(H, W),
                       rel_pos_bias=False, shift_mask=False)
    ref = attention_core(cfg, qkv.float(), (shy, shx), None)
    out = pkg.ops.window_attention(qkv.to(cuda).view(B * H * W, -1), B, (H, W), heads, hd, (wsy, wsx), (shy, shx), None, False)
    out2 = pkg.ops.window_attention(qkv.to(cuda).view(B * H * W, -1), B, (H, W), heads, hd, (wsy, wsx), (shy, shx), None, False)
    torch.cuda.synchronize()
    assert torch.equal(out, out2)
    err = rel_l2(out.view(B, H * W, inner), ref)
    assert err <= 6e-3, err
    assert (out.float().cpu().view(B, H * W, inner) - ref).abs().max() < 0.06


@pytest.mark.parametrize("case", [
    # B, H, W, heads, head_dim, ws, q/k magnitude: logits of +-100 and more in the exp2 domain
    (1, 40, 40, 2, 128, 20, 7.0),
    (1, 60, 60, 1, 128, 60, 9.0),   # the reference's window
    (1, 40, 20, 2, 64, 20, 8.0),
], ids=["ws20_hd128_x7", "ws60_hd128_x9", "ws20_hd64_x8"])
def test_window_attention_streaming_large_logits(pkg, cuda, case):
    """The streaming kernel first sweeps the keys without a row maximum and checks the row sums afterwards; logits that
    overflow exp2 (here: q and k several times larger than N(0,1)) must send the workgroup through the online form and
    give the same softmax.  Bound as for the one-window kernels at this magnitude: q * scale is rounded to bf16 once
    more (as in the reference's bf16 path, model.py:290), a few percent of P once logits reach the hundreds."""
    B, H, W, heads, hd, ws, mag = case
    g = torch.Generator().manual_seed(int(mag * 10) + hd)
    inner = heads * hd
    qkv = torch.randn(B, H * W, 3 * inner, generator=g)
    qkv[..., :2 * inner] *= mag
    qkv = bf(qkv)
    cfg = OracleConfig(dim=inner, heads=heads, head_dim=hd, mlp_dim=inner, window_size=(ws, ws), image_shape=(H, W),
                       rel_pos_bias=False, shift_mask=False)
    ref = attention_core(cfg, qkv.float(), (ws // 2, ws // 2), None)
    out = pkg.ops.window_attention(qkv.to(cuda).view(B * H * W, -1), B, (H, W), heads, hd, (ws, ws), (ws // 2, ws // 2), None, False)
    torch.cuda.synchronize()
    assert bool(torch.isfinite(out).all())
    err = rel_l2(out.view(B, H * W, inner), ref)
    print(f"streaming attention, |q|,|k| x{mag}: rel-L2 {err:.3e}")
    assert err <= 3e-2, err
    # the same queries handed over as head planes that already hold bf16(q * scale * log2 e) (what the model's to_qkv
    # GEMM writes): q is rounded once, and the oracle on exactly those queries is met at the ordinary tolerance
    S = B * H * W
    c = hd ** -0.5 * LOG2E
    raw = torch.randn(B, H * W, 3 * inner, generator=torch.Generator().manual_seed(int(mag * 10) + hd))
    raw[..., :2 * inner] *= mag
    q_dev, kv = bf(raw[..., :inner] * c), bf(raw[..., inner:])
    ref = attention_core(cfg, torch.cat([q_dev.float() / c, kv.float()], dim=-1), (ws // 2, ws // 2), None)
    planes = torch.cat([q_dev, kv], dim=-1).view(S, 3 * heads, hd).permute(1, 0, 2).contiguous().to(cuda)
    out = pkg.ops.window_attention(planes, B, (H, W), heads, hd, (ws, ws), (ws // 2, ws // 2), None, False, head_planes=True,
                                   q_prescaled=True)
    torch.cuda.synchronize()
    err = rel_l2(out.view(B, H * W, inner), ref)
    print(f"streaming attention, |q|,|k| x{mag}, q prescaled: rel-L2 {err:.3e}")
    assert bool(torch.isfinite(out).all()) and err <= 6e-3, err


def test_window_attention_streaming_wide_rows_match_compact(pkg, cuda):
    """head_dim 128 has two streaming forms: K / V straight into LDS by the load unit when every token offset of an
    image's k / v plane fits 32 bits, through registers otherwise.  A [S, 3 * inner] matrix with 388 heads (token
    stride 298 KB, 4.3 GB in all) takes the second; a compact copy of three of its heads takes the first.  Same
    arithmetic in the same order: the outputs must agree bit for bit."""
    H = W = 120
    heads, hd, ws = 388, 128, 60
    S, inner = H * W, heads * hd
    g = torch.Generator(device=cuda).manual_seed(11)
    qkv = torch.empty(S, 3 * inner, dtype=torch.bfloat16, device=cuda)
    for c0 in range(0, 3 * inner, 16384):  # filled in slabs: no 17 GB f32 temporary
        c1 = min(c0 + 16384, 3 * inner)
        qkv[:, c0:c1] = torch.randn(S, c1 - c0, generator=g, device=cuda).to(torch.bfloat16)
    out = pkg.ops.window_attention(qkv, 1, (H, W), heads, hd, (ws, ws), (30, 30), None, False)
    pick = [0, 201, 387]
    cols = torch.cat([torch.arange(c * inner + h * hd, c * inner + (h + 1) * hd) for c in range(3) for h in pick]).to(cuda)
    small = qkv.index_select(1, cols).contiguous()  # [S, 3 * 3 * 128], columns ordered (c h d) like the big one
    out_small = pkg.ops.window_attention(small, 1, (H, W), len(pick), hd, (ws, ws), (30, 30), None, False)
    torch.cuda.synchronize()
    for i, h in enumerate(pick):
        assert torch.equal(out[:, h * hd:(h + 1) * hd], out_small[:, i * hd:(i + 1) * hd]), h
    assert bool(torch.isfinite(out_small.float()).all()) and float(out_small.float().abs().mean()) > 1e-3


HEAD_PLANE_CASES = [
    # B, H, W, heads, hd, ws_y, ws_x, shift, bias, mask -- one-window kernel (small and large grids) and streaming kernel
    (1, 48, 64, 3, 64, 16, 16, 8, True, True),
    (2, 16, 24, 2, 64, 8, 8, 4, True, True),
    (1, 36, 48, 8, 32, 12, 12, 6, True, False),
    (1, 160, 160, 24, 64, 16, 16, 8, True, True),   # the 256x256 GEMM tiles write the planes
    (1, 120, 120, 2, 128, 60, 60, 30, False, False),
    (2, 40, 60, 3, 64, 20, 20, 10, False, False),
]


@pytest.mark.parametrize("case", HEAD_PLANE_CASES, ids=lambda c: f"B{c[0]}_{c[1]}x{c[2]}_h{c[3]}x{c[4]}_ws{c[5]}")
def test_head_plane_layout_is_bit_identical(pkg, cuda, case):
    """The to_qkv GEMM writing one [tokens, head_dim] plane per part and head, and the attention kernels reading
    them, do the same arithmetic as the [tokens, 3*inner] path: planes == columns, attention outputs equal bit for bit."""
    B, H, W, heads, hd, wsy, wsx, sh, has_bias, use_mask = case
    g = torch.Generator().manual_seed(11 * H + W)
    inner, S, K = heads * hd, B * H * W, 128
    x = bf(torch.randn(S, K, generator=g)).to(cuda)
    w = bf(torch.randn(3 * inner, K, generator=g) / math.sqrt(K)).to(cuda)
    bias = bf(0.3 * torch.randn(3 * inner, generator=g)).to(cuda)
    table = bf(0.7 * torch.randn((2 * wsy - 1) * (2 * wsx - 1), heads, generator=g)).to(cuda) if has_bias else None
    qkv = pkg.ops.gemm(x, w, bias)
    planes = pkg.ops.gemm_heads(x, w, bias, hd)
    torch.cuda.synchronize()
    assert planes.shape == (3 * heads, S, hd)
    assert torch.equal(planes.permute(1, 0, 2).reshape(S, 3 * inner), qkv)
    o1 = pkg.ops.window_attention(qkv, B, (H, W), heads, hd, (wsy, wsx), (sh, sh), table, use_mask)
    o2 = pkg.ops.window_attention(planes, B, (H, W), heads, hd, (wsy, wsx), (sh, sh), table, use_mask, head_planes=True)
    torch.cuda.synchronize()
    assert torch.isfinite(o1).all() and torch.equal(o1, o2)


@pytest.mark.parametrize("shape", [(160 * 160, 24, 64), (32 * 64, 4, 32), (24 * 24, 3, 64)], ids=["persistent", "hd32", "small"])
def test_gemm_heads_scales_the_query_planes_in_fp32(pkg, cuda, shape):
    """q_scale / q_planes of gemm_heads: the key and value planes are untouched bit for bit; a query plane is the fp32
    result times the factor, rounded once - within one bf16 ulp of (rounded result) * factor, and for a factor that is a
    power of two exactly equal to it."""
    S, heads, hd = shape
    g = torch.Generator().manual_seed(S + heads)
    inner, K = heads * hd, 128
    x = bf(torch.randn(S, K, generator=g)).to(cuda)
    w = bf(torch.randn(3 * inner, K, generator=g) / math.sqrt(K)).to(cuda)
    bias = bf(0.3 * torch.randn(3 * inner, generator=g)).to(cuda)
    plain = pkg.ops.gemm_heads(x, w, bias, hd)
    for c in (hd ** -0.5 * LOG2E, 0.25):
        scaled = pkg.ops.gemm_heads(x, w, bias, hd, q_scale=c, q_planes=heads)
        torch.cuda.synchronize()
        assert torch.equal(scaled[heads:], plain[heads:])
        want = plain[:heads].float() * c
        if c == 0.25:
            assert torch.equal(scaled[:heads].float(), want)
        else:
            assert bool(((scaled[:heads].float() - want).abs() <= want.abs() * 2.0 ** -7 + 1e-30).all())
            ref = (x.float() @ w[:inner].float().T + bias[:inner].float()) * c  # fp32 throughout, one rounding at the end
            got = scaled[:heads].permute(1, 0, 2).reshape(S, inner).float()
            assert rel_l2(got.cpu(), ref.cpu()) <= 2.5e-3  # one bf16 rounding: 2^-9 / sqrt(3) = 1.1e-3 on average


FUSED_CASES = [
    # B, H, W, heads, K, shift, bias + mask, projection bias -- 16x16 windows, head_dim 64: the fused to_qkv + attention kernel
    (1, 160, 160, 24, 1536, 8, True, True),    # configs[3] widths: 24 k-tiles, 2400 units
    (1, 160, 160, 24, 256, 0, False, False),   # 4 k-tiles, no bias anywhere: accumulators start at a literal zero
    (2, 96, 160, 6, 384, 8, True, False),      # two batch entries, 120 windows x 6 heads
    (1, 48, 80, 3, 256, 8, True, True),        # 15 windows (the last group of 4 is short), 4 k-tiles (the fewest), 45 units < 256 workgroups
    (1, 32, 32, 2, 640, 8, True, True),        # every window on the wrapped border; 8 units
]


@pytest.mark.parametrize("case", FUSED_CASES, ids=lambda c: f"B{c[0]}_{c[1]}x{c[2]}_h{c[3]}_K{c[4]}_s{c[5]}_b{int(c[6])}_pb{int(c[7])}")
def test_fused_qkv_window_attention(pkg, cuda, case):
    """The to_qkv projection inside the attention kernel (q, k, v never in HBM) against the two-kernel path (GEMM writing
    head planes with q scaled in its epilogue, then the attention kernel): the same arithmetic in the same order, so
    bit-identical wherever the GEMM of the two-kernel path is the 256x256-tile kernel (same MFMA shape and k order), and
    within the ordinary tolerance of the fp32 oracle everywhere."""
    B, H, W, heads, K, sh, bias_mask, proj_bias = case
    hd, ws = 64, 16
    g = torch.Generator().manual_seed(H * W + heads + K)
    inner, S = heads * hd, B * H * W
    y = bf(torch.randn(S, K, generator=g))
    w = bf(torch.randn(3 * inner, K, generator=g) / math.sqrt(K))
    pb = bf(0.3 * torch.randn(3 * inner, generator=g)) if proj_bias else None
    table = bf(0.7 * torch.randn((2 * ws - 1) ** 2, heads, generator=g)) if bias_mask else None
    ops = pkg.ops
    assert ops.qkv_attention_supported(K, heads, hd, (ws, ws), (H, W))
    yd, wd = y.to(cuda), w.to(cuda)
    pbd = None if pb is None else pb.to(cuda)
    td = None if table is None else table.to(cuda)
    b4 = None if td is None else ops.qkv_attention_pack_bias(td, (ws, ws))
    got = ops.qkv_window_attention(yd, wd, pbd, b4, B, (H, W), heads, hd, (ws, ws), (sh, sh), bias_mask)
    got2 = ops.qkv_window_attention(yd, wd, pbd, b4, B, (H, W), heads, hd, (ws, ws), (sh, sh), bias_mask)
    planes = ops.gemm_heads(yd, wd, pbd, hd, q_scale=hd ** -0.5 * LOG2E, q_planes=heads)
    two = ops.window_attention(planes, B, (H, W), heads, hd, (ws, ws), (sh, sh), td, bias_mask, head_planes=True,
                               q_prescaled=True)
    torch.cuda.synchronize()
    assert torch.equal(got, got2) and bool(torch.isfinite(got.float()).all())
    if ops.gemm_uses_big_tiles(S, 3 * inner):
        assert torch.equal(got, two)
    else:
        assert rel_l2(got, two) <= 4e-3, rel_l2(got, two)
    cfg = OracleConfig(dim=inner, heads=heads, head_dim=hd, mlp_dim=inner, window_size=(ws, ws), image_shape=(H, W),
                       rel_pos_bias=bias_mask, shift_mask=bias_mask)
    qkv = y.float() @ w.float().T + (0 if pb is None else pb.float())
    ref = attention_core(cfg, qkv.view(B, H * W, 3 * inner), (sh, sh), None if table is None else table.float())
    err = rel_l2(got.view(B, H * W, inner), ref)
    print(f"fused qkv + attention {case}: rel-L2 vs fp32 oracle {err:.3e}")
    assert err <= 6e-3, err


def test_fused_qkv_window_attention_rejects_other_shapes(pkg, cuda):
    ops = pkg.ops
    assert not ops.qkv_attention_supported(1536, 24, 64, (12, 12), (180, 360))
    assert not ops.qkv_attention_supported(1536, 12, 128, (16, 16), (160, 160))
    assert not ops.qkv_attention_supported(1472, 24, 64, (16, 16), (160, 160))  # K % 128
    assert not ops.qkv_attention_supported(128, 2, 64, (16, 16), (160, 160))  # fewer than 4 k-tiles
    y = torch.zeros(144 * 4, 128, dtype=torch.bfloat16, device=cuda)
    w = torch.zeros(3 * 64, 128, dtype=torch.bfloat16, device=cuda)
    with pytest.raises(pkg.AerisError) as e:
        ops.qkv_window_attention(y, w, None, None, 1, (24, 24), 1, 64, (12, 12))
    assert e.value.code == -2


NONFINITE_CASES = [
    # B, H, W, heads, hd, ws, shift, bias + mask, head planes -- one case per kernel form
    ("persistent", 1, 160, 160, 24, 64, 16, 8, True, True),
    ("one_unit_dma", 3, 32, 48, 2, 64, 16, 8, True, True),
    ("register_staged_rows", 1, 48, 64, 3, 64, 16, 8, True, False),
    ("register_staged_hd32", 1, 32, 64, 4, 32, 8, 4, True, True),
    ("streaming_rows", 2, 40, 60, 3, 64, 20, 10, False, False),
    ("streaming_planes_hd128", 1, 120, 120, 2, 128, 60, 30, False, True),
]


@pytest.mark.parametrize("case", NONFINITE_CASES, ids=lambda c: c[0])
def test_window_attention_non_finite_inputs_stay_in_their_window(pkg, cuda, case):
    """NaN-in -> NaN-out, and nowhere else.  One token's q, k, v (all heads) are NaN and another token's, in a different
    window, +Inf.  The kernels' fast path (no row maximum) sees row sums out of range and repeats the window in the
    two-pass / online form; the call returns, every output of the NaN window is NaN (its key poisons every query's
    softmax), every output of the Inf window is non-finite (Inf - Inf in the logits), and every other window is bit for
    bit what it is on clean inputs."""
    _, B, H, W, heads, hd, ws, sh, bias_mask, planes = case
    g = torch.Generator().manual_seed(H + W + hd)
    inner, S = heads * hd, B * H * W
    qkv = bf(torch.randn(S, 3 * inner, generator=g))
    table = bf(0.7 * torch.randn((2 * ws - 1) ** 2, heads, generator=g)).to(cuda) if bias_mask else None
    wmap = torch.from_numpy(pkg.ops.window_index_map(B, H, W, ws, ws, sh, sh))  # [windows, L] token rows
    n_win = wmap.shape[0]
    w_nan, w_inf = n_win - 1, n_win // 2  # the last window lies on the wrapped, masked border of a shifted grid
    bad = qkv.clone()
    bad[wmap[w_nan, 5]] = float("nan")
    bad[wmap[w_inf, wmap.shape[1] - 3]] = float("inf")

    def run(t):
        if planes:
            t = t.view(S, 3 * heads, hd).permute(1, 0, 2).contiguous()
        else:
            t = t.view(S, 3 * inner)
        return pkg.ops.window_attention(t.to(cuda), B, (H, W), heads, hd, (ws, ws), (sh, sh), table, bias_mask,
                                        head_planes=planes)

    clean, got = run(qkv), run(bad)
    torch.cuda.synchronize()  # returns: no wave spins on a value that never becomes finite
    assert bool(torch.isfinite(clean.float()).all())
    rows_nan, rows_inf = wmap[w_nan].to(cuda), wmap[w_inf].to(cuda)
    assert bool(torch.isnan(got[rows_nan].float()).all())
    assert not bool(torch.isfinite(got[rows_inf].float()).any())
    keep = torch.ones(S, dtype=torch.bool, device=cuda)
    keep[rows_nan] = False
    keep[rows_inf] = False
    assert torch.equal(got[keep], clean[keep])


def test_window_attention_streaming_rejects_bias_and_mask(pkg, cuda):
    qkv = torch.zeros(60 * 60, 3 * 128, dtype=torch.bfloat16, device=cuda)
    table = torch.zeros(119 * 119, 1, dtype=torch.bfloat16, device=cuda)
    with pytest.raises(pkg.AerisError) as e:
        pkg.ops.window_attention(qkv, 1, (60, 60), 1, 128, (60, 60), (0, 0), table, False)
    assert e.value.code == -2
    with pytest.raises(pkg.AerisError) as e:
        pkg.ops.window_attention(qkv, 1, (60, 60), 1, 128, (60, 60), (30, 30), None, True)
    assert e.value.code == -2


@pytest.mark.parametrize("geo", [(2, 32, 64, 8, 4), (1, 36, 60, 12, 6), (1, 48, 80, 16, 8), (1, 32, 32, 16, 0)])
@pytest.mark.parametrize("disp", [(0, 0), (0, -1), (1, 0), (-2, 3)])
def test_attention_index_map_bit_exact(pkg, cuda, geo, disp):
    """q = k = 0 and a bias table that is 0 at one displacement and -30000 elsewhere make every query copy the
    value of exactly one key, so the output must equal, bit for bit, v gathered through the oracle's
    partition + roll map (and scattered back through it)."""
    B, H, W, ws, sh = geo
    heads, hd = 2, 64
    inner = heads * hd
    dy, dx = disp
    g = torch.Generator().manual_seed(7)
    v = bf(torch.randn(B * H * W, inner, generator=g))
    qkv = torch.zeros(B * H * W, 3 * inner, dtype=torch.bfloat16)
    qkv[:, 2 * inner:] = v
    table = torch.full(((2 * ws - 1) ** 2, heads), -30000.0)
    table[(dy + ws - 1) * (2 * ws - 1) + (dx + ws - 1)] = 0.0  # relative index of (query - key) = (dy, dx)
    out = pkg.ops.window_attention(qkv.to(cuda), B, (H, W), heads, hd, (ws, ws), (sh, sh), bf(table).to(cuda), False)
    torch.cuda.synchronize()
    out = out.cpu()
    idx = oracle.window_token_index(B, H, W, ws, ws, sh, sh)  # [nW, L]
    checked = 0
    for p in range(ws * ws):
        ky, kx = p // ws - dy, p % ws - dx  # the key this query selects
        if 0 <= ky < ws and 0 <= kx < ws:
            q_rows, k_rows = idx[:, p], idx[:, ky * ws + kx]
            assert torch.equal(out[q_rows], v[k_rows]), (p, disp)
            checked += 1
    assert checked >= (ws - 3) * (ws - 3)


def test_attention_uniform_v_and_determinism_full_grid(pkg, cuda):
    """configs[2] size (720x1440, 16 heads x 64, 16x16 windows, shift 8): uniform V per window => out = V;
    two launches agree bit for bit; sampled windows match the oracle."""
    B, H, W, heads, hd, ws, sh = 1, 720, 1440, 16, 64, 16, 8
    inner = heads * hd
    S = H * W
    g = torch.Generator(device="cuda").manual_seed(3)
    qkv = torch.randn(S, 3 * inner, generator=g, device=cuda, dtype=torch.float32).to(torch.bfloat16)
    table = (0.5 * torch.randn((2 * ws - 1) ** 2, heads, generator=g, device=cuda)).to(torch.bfloat16)
    out1 = pkg.ops.window_attention(qkv, B, (H, W), heads, hd, (ws, ws), (sh, sh), table, True)
    out2 = pkg.ops.window_attention(qkv, B, (H, W), heads, hd, (ws, ws), (sh, sh), table, True)
    torch.cuda.synchronize()
    assert torch.equal(out1, out2)
    # sampled windows (first, a middle one, last row / last column / corner: the masked ones)
    idx_all = oracle.window_token_index(B, H, W, ws, ws, sh, sh)
    nWx = W // ws
    picks = [0, 17 * nWx + 33, 44 * nWx + 5, 20 * nWx + (nWx - 1), 44 * nWx + nWx - 1]
    ridx = torch.from_numpy(oracle.relative_position_index(ws, ws))
    bias = table.float().cpu()[ridx.reshape(-1)].reshape(ws * ws, ws * ws, heads).permute(2, 0, 1)
    mask_all = oracle.shift_attention_mask(H, W, ws, ws, sh, sh)
    for w in picks:
        rows = torch.from_numpy(idx_all[w])
        win = qkv[rows.to(cuda)].float().cpu().reshape(ws * ws, 3, heads, hd)
        q, k, v = (win[:, c].permute(1, 0, 2)[None] for c in range(3))
        ref = oracle.window_attention(q, k, v, hd ** -0.5, bias, torch.from_numpy(mask_all[w])[None])
        got = out1[rows.to(cuda)].float().cpu().reshape(ws * ws, heads, hd).permute(1, 0, 2)[None]
        assert rel_l2(got, ref) <= 6e-3, w
    # uniform V inside every window (value depends on the window only) => output equals V
    win_of_token = torch.empty(S, dtype=torch.int64)
    win_of_token[torch.from_numpy(idx_all.reshape(-1))] = torch.arange(idx_all.shape[0]).repeat_interleave(ws * ws)
    vals = torch.randn(idx_all.shape[0], inner, generator=torch.Generator().manual_seed(5)).to(torch.bfloat16)
    qkv[:, 2 * inner:] = vals[win_of_token].to(cuda)
    out = pkg.ops.window_attention(qkv, B, (H, W), heads, hd, (ws, ws), (sh, sh), table, True)
    torch.cuda.synchronize()
    diff = (out.float() - qkv[:, 2 * inner:].float()).abs().max().item()
    assert diff <= 0.04, diff  # sum of bf16-rounded probabilities differs from the fp32 row sum by < 2^-8 relative


# ---------------------------------------------------------------------------------------------- norm + modulation

@pytest.mark.parametrize("d", [128, 512, 1024, 1536, 2048, 3072])
@pytest.mark.parametrize("kind,order", [("layernorm", "norm_then_mod"), ("rmsnorm", "mod_then_norm"), ("layernorm", "mod_then_norm"), ("rmsnorm", "norm_then_mod")])
@pytest.mark.parametrize("xdt", [torch.bfloat16, torch.float32])
def test_norm_modulate_parity(pkg, cuda, d, kind, order, xdt):
    B, S = 3, 333
    g = torch.Generator().manual_seed(d)
    x = (1.5 * torch.randn(B, S, d, generator=g) + 0.3).to(xdt)
    gamma, beta = bf(1 + 0.2 * torch.randn(d, generator=g)), bf(0.2 * torch.randn(d, generator=g))
    mods = 0.3 * torch.randn(B, 2 * d, generator=g)  # strided chunks of one wider matrix, like the block uses them
    shift, scale = mods[:, :d], mods[:, d:]
    eps = 1e-5 if kind == "layernorm" else float(torch.finfo(torch.float32).eps)
    xf = x.float()

    def norm(v):
        if kind == "layernorm":
            return oracle.layer_norm(v, gamma.float(), beta.float(), eps)
        return oracle.rms_norm(v, gamma.float(), eps)

    ref = norm(oracle.modulate(xf, shift, scale)) if order == "mod_then_norm" else oracle.modulate(norm(xf), shift, scale)
    md = mods.to(cuda)
    out = pkg.ops.norm_modulate(x.to(cuda), gamma.to(cuda), beta.to(cuda) if kind == "layernorm" else None,
                                md[:, :d], md[:, d:], kind=kind, order=order, eps=eps)
    torch.cuda.synchronize()
    assert rel_l2(out, ref) <= 3e-3
    out32 = pkg.ops.norm_modulate(x.to(cuda), gamma.to(cuda), beta.to(cuda) if kind == "layernorm" else None,
                                  md[:, :d], md[:, d:], kind=kind, order=order, eps=eps, out_dtype=torch.float32)
    assert rel_l2(out32, ref) <= 1e-5


def test_norm_modulate_variants(pkg, cuda):
    d, B, S = 512, 2, 50
    g = torch.Generator().manual_seed(1)
    x = torch.randn(B, S, d, generator=g)
    gamma32, beta32 = 1 + 0.2 * torch.randn(d, generator=g), 0.2 * torch.randn(d, generator=g)
    # f32 parameters, no modulation
    out = pkg.ops.norm_modulate(x.to(cuda), gamma32.to(cuda), beta32.to(cuda), kind="layernorm", out_dtype=torch.float32)
    assert rel_l2(out, oracle.layer_norm(x, gamma32, beta32, 1e-5)) <= 1e-5
    # one modulation row broadcast over the batch; shift only (scale None => x + shift, model.py:122-123)
    sh = torch.randn(1, d, generator=g)
    out = pkg.ops.norm_modulate(x.to(cuda), gamma32.to(cuda), None, sh.to(cuda), None, kind="rmsnorm",
                                order="mod_then_norm", eps=1e-6, out_dtype=torch.float32)
    assert rel_l2(out, oracle.rms_norm(oracle.modulate(x, sh, None), gamma32, 1e-6)) <= 1e-5
    # a single row, and a row count that is not a multiple of the block's 4 waves
    x1 = torch.randn(1, 1, d, generator=g)
    out = pkg.ops.norm_modulate(x1.to(cuda), gamma32.to(cuda), beta32.to(cuda), out_dtype=torch.float32)
    assert rel_l2(out, oracle.layer_norm(x1, gamma32, beta32, 1e-5)) <= 1e-5


# ---------------------------------------------------------------------------------------------- small ops

@pytest.mark.parametrize("wdt", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("B", [1, 4, 9])
def test_modulation_linear_parity(pkg, cuda, wdt, B):
    d = 384
    g = torch.Generator().manual_seed(B)
    t = torch.randn(B, d, generator=g)
    w0, b0 = (torch.randn(d, d, generator=g) / math.sqrt(d)).to(wdt), (0.1 * torch.randn(d, generator=g)).to(wdt)
    w2, b2 = (torch.randn(6 * d, d, generator=g) / math.sqrt(d)).to(wdt), (0.1 * torch.randn(6 * d, generator=g)).to(wdt)
    ref = oracle.modulation_mlp(t, w0.float(), b0.float(), w2.float(), b2.float())
    h = pkg.ops.modulation_linear(t.to(cuda), w0.to(cuda), b0.to(cuda), silu=True)
    out = pkg.ops.modulation_linear(h, w2.to(cuda), b2.to(cuda))
    torch.cuda.synchronize()
    assert rel_l2(out, ref) <= 1e-5


def test_timestep_embedding_parity(pkg, cuda):
    t = torch.tensor([0.0, 0.3, math.pi / 2, 1.2])
    for dim in (128, 1536):
        out = pkg.ops.timestep_embedding(t.to(cuda), dim, 10_000.0)
        ref = oracle.timestep_embedding(t.double(), dim, 10_000)
        assert (out.double().cpu() - ref).abs().max() < 2e-6
    out0 = pkg.ops.timestep_embedding(torch.zeros(1, device=cuda), 64)
    assert torch.equal(out0[0, :32].cpu(), torch.zeros(32)) and torch.equal(out0[0, 32:].cpu(), torch.ones(32))


def test_embed_prepare_parity(pkg, cuda):
    g = torch.Generator().manual_seed(2)
    B, S, C = 2, 300, 138
    x, ape = torch.randn(B * S, C, generator=g), torch.randn(S, C, generator=g)
    out = pkg.ops.embed_prepare(x.to(cuda), ape.to(cuda), 192).cpu()
    ref = torch.zeros(B * S, 192)
    ref[:, :C] = x + ape.repeat(B, 1)
    assert torch.equal(out, ref.to(torch.bfloat16))
    out = pkg.ops.embed_prepare(x.to(cuda), None, 192).cpu()
    ref[:, :C] = x
    assert torch.equal(out, ref.to(torch.bfloat16))


def test_embed_prepare_split_layout(pkg, cuda):
    """split: every value v is written as [hi | lo | hi | 1 | 1], hi = bf16(v), lo = bf16(v - hi), zero padded: hi + lo
    reproduces v to 2^-16 relative, and the concatenating form writes the same."""
    g = torch.Generator().manual_seed(4)
    M, C, K = 500, 138, 448
    x, ape = torch.randn(M, C, generator=g) * 3, torch.randn(100, C, generator=g)
    out = pkg.ops.embed_prepare(x.to(cuda), ape.to(cuda), K, split=True).cpu()
    v = x + ape.repeat(5, 1)
    hi = v.to(torch.bfloat16)
    lo = (v - hi.float()).to(torch.bfloat16)
    assert torch.equal(out[:, :C], hi) and torch.equal(out[:, C:2 * C], lo) and torch.equal(out[:, 2 * C:3 * C], hi)
    assert torch.equal(out[:, 3 * C:3 * C + 2].float(), torch.ones(M, 2)) and not out[:, 3 * C + 2:].any()
    assert float(((hi.float() + lo.float()) - v).abs().max() / v.abs().max()) < 2.0 ** -15
    got = pkg.ops.embed_concat(x[:, :69].contiguous().to(cuda), 1.0, x[:, 69:].contiguous().to(cuda), ape.to(cuda), K,
                               split=True).cpu()
    assert torch.equal(got, out)


def test_embed_concat_equals_cat_then_prepare(pkg, cuda):
    """The sampler's cat([x_t / sigma_d, conditioning], 2) (inference.py:160) folded into the operand preparation
    is bit-identical to concatenating first."""
    g = torch.Generator().manual_seed(3)
    B, S, C0, C1 = 2, 300, 69, 69
    x0, x1, ape = torch.randn(B * S, C0, generator=g), torch.randn(B * S, C1, generator=g), torch.randn(S, C0 + C1, generator=g)
    for div0 in (1.0, 0.5, 1.7):
        for a in (ape, None):
            ref = pkg.ops.embed_prepare(torch.cat([x0 / div0, x1], dim=1).to(cuda), None if a is None else a.to(cuda), 192)
            got = pkg.ops.embed_concat(x0.to(cuda), div0, x1.to(cuda), None if a is None else a.to(cuda), 192)
            assert torch.equal(got, ref), (div0, a is None)
    # uneven split
    got = pkg.ops.embed_concat(x0[:, :5].contiguous().to(cuda), 2.0, x1.to(cuda), None, 128)
    ref = pkg.ops.embed_prepare(torch.cat([x0[:, :5] / 2.0, x1], dim=1).to(cuda), None, 128)
    assert torch.equal(got, ref)
