"""Pin the oracle's floating-point pieces against torch library modules, closed forms, float64
loops and invariants.  The reference holds no test vectors for this path, so these are the pins.
"""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

import oracle
from oracle import OracleConfig
from oracle.swin_oracle import attention_core

torch.manual_seed(0)


def test_norms_match_torch_library():
    x = torch.randn(3, 7, 48)
    g, b = torch.randn(48), torch.randn(48)
    torch.testing.assert_close(oracle.layer_norm(x, g, b, 1e-5), F.layer_norm(x, (48,), g, b, 1e-5), rtol=1e-5, atol=1e-5)
    rn = torch.nn.RMSNorm(48)  # eps=None, as at model.py:387
    with torch.no_grad():
        rn.weight.copy_(g)
    torch.testing.assert_close(oracle.rms_norm(x, g, torch.finfo(torch.float32).eps), rn(x), rtol=1e-5, atol=1e-6)
    # closed form on a constant row: LN -> beta, RMS -> sign * gamma
    c = torch.full((1, 1, 48), 3.0)
    torch.testing.assert_close(oracle.layer_norm(c, g, b, 1e-5), b.expand(1, 1, 48), rtol=0, atol=1e-6)
    torch.testing.assert_close(oracle.rms_norm(c, g, 0.0), g.expand(1, 1, 48), rtol=1e-6, atol=1e-6)


def test_modulate_closed_form():
    x = torch.randn(2, 5, 8)
    sh, sc = torch.randn(2, 8), torch.randn(2, 8)
    got = oracle.modulate(x, sh, sc)
    for b in range(2):
        for s in range(5):
            torch.testing.assert_close(got[b, s], x[b, s] * (1 + sc[b]) + sh[b])
    torch.testing.assert_close(oracle.modulate(x, sh, None), x + sh[:, None, :])


def test_modulation_mlp_matches_torch_sequential():
    d = 16
    seq = torch.nn.Sequential(torch.nn.Linear(d, d), torch.nn.SiLU(), torch.nn.Linear(d, 6 * d))
    t = torch.randn(2, d)
    got = oracle.modulation_mlp(t, seq[0].weight, seq[0].bias, seq[2].weight, seq[2].bias)
    torch.testing.assert_close(got, seq(t), rtol=1e-5, atol=1e-6)


def test_timestep_embedding_known_answers():
    d = 32
    e0 = oracle.timestep_embedding(torch.zeros(1), d)
    torch.testing.assert_close(e0[0, :16], torch.zeros(16))  # sin half first (after the flip, model.py:139-141)
    torch.testing.assert_close(e0[0, 16:], torch.ones(16))
    t = torch.tensor([0.3, math.pi / 2], dtype=torch.float64)
    e = oracle.timestep_embedding(t, d, 10_000)
    for b in range(2):
        for k in range(16):
            f = math.exp(-math.log(10_000) * k / 16)
            assert abs(e[b, k].item() - math.sin(t[b].item() * f)) < 1e-12
            assert abs(e[b, 16 + k].item() - math.cos(t[b].item() * f)) < 1e-12
    # the same through the reference's route: cat[cos, sin] then swap the halves
    args = t[:, None] * torch.exp(-math.log(10_000) * torch.arange(16, dtype=torch.float64) / 16)[None]
    route = torch.cat([torch.cos(args), torch.sin(args)], -1).reshape(2, 2, -1).flip(1).reshape(2, d)
    torch.testing.assert_close(e, route, rtol=0, atol=0)


def test_positional_encoding_2d_closed_form():
    C, h, w = 10, 5, 7
    pe = oracle.positional_encoding_2d(C, h, w)
    ch = int(math.ceil(C / 4) * 2)  # 6
    assert pe.shape == (h, w, C)
    torch.testing.assert_close(pe[0, 0, :ch], torch.tensor([0., 1., 0., 1., 0., 1.]))
    for y in range(h):
        for x in range(w):
            for c in range(C):
                pos, cc = (y, c) if c < ch else (x, c - ch)  # first ch channels encode the ROW (model.py:183)
                f = 1.0 / (10_000 ** ((cc // 2 * 2) / ch))
                want = math.sin(pos * f) if cc % 2 == 0 else math.cos(pos * f)
                assert abs(pe[y, x, c].item() - want) < 1e-5


def _attention_loops64(q, k, v, scale, bias, mask):
    nW, h, L, hd = q.shape
    out = np.zeros((nW, h, L, hd))
    q, k, v = q.double().numpy(), k.double().numpy(), v.double().numpy()
    for w in range(nW):
        for j in range(h):
            for p in range(L):
                s = np.array([scale * float(q[w, j, p] @ k[w, j, r]) for r in range(L)])
                if bias is not None:
                    s = s + bias[j, p].double().numpy()
                if mask is not None:
                    s = s + mask[w, p].double().numpy()
                e = np.exp(s - s.max())
                out[w, j, p] = (e / e.sum()) @ v[w, j]
    return out


def test_window_attention_vs_float64_loops_and_sdpa():
    nW, h, L, hd = 3, 2, 6, 4
    q, k, v = torch.randn(nW, h, L, hd), torch.randn(nW, h, L, hd), torch.randn(nW, h, L, hd)
    bias = torch.randn(h, L, L)
    mask = torch.where(torch.rand(nW, L, L) > 0.7, -100.0, 0.0)
    mask[:, torch.arange(L), torch.arange(L)] = 0.0
    got = oracle.window_attention(q, k, v, hd ** -0.5, bias, mask)
    want = _attention_loops64(q, k, v, hd ** -0.5, bias, mask)
    np.testing.assert_allclose(got.numpy(), want, rtol=1e-5, atol=1e-6)
    sdpa = F.scaled_dot_product_attention(q, k, v, attn_mask=bias[None] + mask[:, None])
    torch.testing.assert_close(got, sdpa, rtol=1e-5, atol=1e-6)
    plain = oracle.window_attention(q, k, v, hd ** -0.5)
    torch.testing.assert_close(plain, F.scaled_dot_product_attention(q, k, v), rtol=1e-5, atol=1e-6)


def test_window_attention_invariants():
    nW, h, L, hd = 2, 2, 9, 4
    q, k = torch.randn(nW, h, L, hd), torch.randn(nW, h, L, hd)
    v = torch.randn(nW, h, 1, hd).expand(nW, h, L, hd)
    out = oracle.window_attention(q, k, v, 0.5)
    torch.testing.assert_close(out, v.contiguous(), rtol=1e-5, atol=1e-6)  # uniform V => output = V
    v = torch.randn(nW, h, L, hd)
    perm = torch.randperm(L)
    a = oracle.window_attention(q, k, v, 0.5)
    b = oracle.window_attention(q[:, :, perm], k[:, :, perm], v[:, :, perm], 0.5)
    torch.testing.assert_close(a[:, :, perm], b, rtol=1e-5, atol=1e-6)  # permutation equivariance


@pytest.mark.parametrize("shift", [(0, 0), (2, 2), (1, 3)])
def test_attention_core_equals_gather_attend_scatter(shift):
    """Un-fused roll/partition/reverse/roll path == gather by the folded index map, attend, scatter back."""
    cfg = OracleConfig(dim=16, heads=2, head_dim=4, mlp_dim=32, window_size=(4, 4), image_shape=(8, 12),
                       rel_pos_bias=True, shift_mask=True)
    B, (H, W), (wy, wx) = 2, cfg.image_shape, cfg.window_size
    S, inner = H * W, cfg.inner
    qkv = torch.randn(B, S, 3 * inner)
    table = torch.randn((2 * wy - 1) * (2 * wx - 1), cfg.heads)
    got = attention_core(cfg, qkv, shift, table, window_chunk=3)
    idx = torch.from_numpy(oracle.window_token_index(B, H, W, wy, wx, *shift))  # [nW, L]
    flat = qkv.reshape(B * S, 3, cfg.heads, cfg.head_dim)
    win = flat[idx]  # [nW, L, 3, h, hd]
    q, k, v = (win[:, :, c].permute(0, 2, 1, 3) for c in range(3))
    ridx = torch.from_numpy(oracle.relative_position_index(wy, wx))
    bias = table[ridx.reshape(-1)].reshape(wy * wx, wy * wx, cfg.heads).permute(2, 0, 1)
    mask = None
    if shift != (0, 0):
        mask = torch.from_numpy(oracle.shift_attention_mask(H, W, wy, wx, *shift)).repeat(B, 1, 1)
    o = oracle.window_attention(q, k, v, cfg.head_dim ** -0.5, bias, mask)  # [nW, h, L, hd]
    want = torch.empty(B * S, inner)
    want[idx.reshape(-1)] = o.permute(0, 2, 1, 3).reshape(-1, inner)
    torch.testing.assert_close(got.reshape(B * S, inner), want, rtol=1e-5, atol=1e-6)


def test_mlps_match_torch_library():
    d, Hd = 16, 40
    z = torch.randn(2, 5, d)
    cfg = OracleConfig.ref(dim=d, heads=2, head_dim=8, mlp_dim=Hd, window_size=(2, 2), image_shape=(2, 2))
    sd = oracle.init_block_weights(cfg, 1, nontrivial=True)
    gu = F.linear(z, sd["modulelist.0.3.w1.weight"])
    want = F.linear(F.silu(gu[..., :Hd]) * gu[..., Hd:], sd["modulelist.0.3.w2.weight"])  # gate first (model.py:157)
    torch.testing.assert_close(oracle.mlp_branch(cfg, sd, "modulelist.0.", z), want, rtol=1e-5, atol=1e-6)
    cfg = OracleConfig.spec(dim=d, heads=2, head_dim=8, mlp_dim=Hd, window_size=(2, 2), image_shape=(2, 2))
    sd = oracle.init_block_weights(cfg, 1, nontrivial=True)
    p = "modulelist.0.3."
    want = F.linear(F.gelu(F.linear(z, sd[p + "fc1.weight"], sd[p + "fc1.bias"])), sd[p + "fc2.weight"], sd[p + "fc2.bias"])
    torch.testing.assert_close(oracle.mlp_branch(cfg, sd, "modulelist.0.", z), want, rtol=1e-5, atol=1e-6)


def _cfgs():
    geo = dict(dim=32, heads=2, head_dim=8, mlp_dim=64, window_size=(4, 4), image_shape=(8, 8))
    return {"ref": OracleConfig.ref(**geo), "spec": OracleConfig.spec(mod_ways=3, **geo),
            "spec2": OracleConfig.spec(mod_ways=2, **geo), "spec0": OracleConfig.spec(mod_ways=0, **geo)}


@pytest.mark.parametrize("name", ["ref", "spec"])
def test_block_is_identity_when_gates_are_zero(name):
    cfg = _cfgs()[name]
    sd = oracle.init_block_weights(cfg, 3, nontrivial=True)
    d = cfg.dim
    for k in ("weight", "bias"):
        sd[f"modulelist.0.4.modulation.2.{k}"][2 * d:3 * d] = 0
        sd[f"modulelist.0.4.modulation.2.{k}"][5 * d:6 * d] = 0
    x, t = torch.randn(2, 64, d), torch.randn(1, d)
    torch.testing.assert_close(oracle.block_forward(cfg, sd, x, t, (2, 2)), x, rtol=0, atol=0)


@pytest.mark.parametrize("name", ["ref", "spec"])
def test_block_reduces_to_plain_prenorm_block(name):
    """gate = 1, shift = scale = 0  =>  x + attn(norm(x)); then + mlp(norm(.)), built from torch library ops."""
    cfg = _cfgs()[name]
    sd = oracle.init_block_weights(cfg, 4, nontrivial=True)
    d = cfg.dim
    sd["modulelist.0.4.modulation.2.weight"].zero_()
    b2 = torch.zeros(6 * d)
    b2[2 * d:3 * d] = 1
    b2[5 * d:] = 1
    sd["modulelist.0.4.modulation.2.bias"] = b2
    x, t = torch.randn(1, 64, d), torch.randn(1, d)
    got = oracle.block_forward(cfg, sd, x, t, (0, 0))
    p = "modulelist.0."

    def norm(n, v):
        if cfg.norm == "layernorm":
            return F.layer_norm(v, (d,), sd[f"{p}{n}.weight"], sd[f"{p}{n}.bias"], 1e-5)
        return F.rms_norm(v, (d,), sd[f"{p}{n}.weight"], torch.finfo(torch.float32).eps)

    x1 = x + oracle.attention_branch(cfg, sd, p, norm("0", x), (0, 0))
    want = x1 + oracle.mlp_branch(cfg, sd, p, norm("2", x1))
    torch.testing.assert_close(got, want, rtol=1e-5, atol=1e-5)


def test_modulation_order_and_chunk_order():
    """REF: norm(modulate(x)); SPEC: modulate(norm(x)); chunks are shift, scale, gate per branch (model.py:399)."""
    for name in ("ref", "spec"):
        cfg = _cfgs()[name]
        d = cfg.dim
        sd = oracle.init_block_weights(cfg, 5, nontrivial=True)
        x, t = torch.randn(1, 64, d), torch.randn(1, d)
        m = oracle.modulation_mlp(t, *(sd[f"modulelist.0.4.modulation.{i}.{k}"] for i in (0, 2) for k in ("weight", "bias")))
        s1, c1, g1, s2, c2, g2 = m.chunk(6, dim=1)
        p = "modulelist.0."
        if cfg.norm == "layernorm":
            nrm = lambda n, v: F.layer_norm(v, (d,), sd[f"{p}{n}.weight"], sd[f"{p}{n}.bias"], 1e-5)
        else:
            nrm = lambda n, v: F.rms_norm(v, (d,), sd[f"{p}{n}.weight"], torch.finfo(torch.float32).eps)
        if cfg.mod_order == "mod_then_norm":
            y = nrm("0", x * (1 + c1[:, None]) + s1[:, None])
        else:
            y = nrm("0", x) * (1 + c1[:, None]) + s1[:, None]
        x1 = x + g1[:, None] * oracle.attention_branch(cfg, sd, p, y, (2, 2))
        if cfg.mod_order == "mod_then_norm":
            z = nrm("2", x1 * (1 + c2[:, None]) + s2[:, None])
        else:
            z = nrm("2", x1) * (1 + c2[:, None]) + s2[:, None]
        want = x1 + g2[:, None] * oracle.mlp_branch(cfg, sd, p, z)
        got, a, mo = oracle.block_forward(cfg, sd, x, t, (2, 2), return_branches=True)
        torch.testing.assert_close(got, want, rtol=1e-5, atol=1e-5)
        assert (got - x).abs().max() > 1e-2  # the gates are open in this init: the comparison is not vacuous


def test_model_folded_shift_equals_rolling_the_residual_stream():
    """model.py:470-475 rolls the residual stream around odd layers; the oracle shifts only inside
    attention.  Both must agree because everything else in a block is pointwise per token."""
    geo = dict(dim=32, heads=2, head_dim=8, mlp_dim=64, window_size=(4, 4), image_shape=(8, 8))
    cfg = OracleConfig.ref(n_layers=5, in_channels=6, out_channels=3, **geo)
    sd = oracle.init_model_weights(cfg, 1, nontrivial=True)
    x, dt = torch.randn(1, 64, 6), torch.tensor([0.7])
    got = oracle.model_forward(cfg, sd, x, dt)
    tok, t = oracle.input_stage(cfg, sd, x, dt)
    for i in range(cfg.n_layers - 2):
        if i % 2 == 1:
            tok = torch.roll(tok.reshape(1, 8, 8, -1), (-2, -2), (1, 2)).reshape(1, 64, -1)
        tok = oracle.block_forward(cfg, sd, tok, t, (0, 0), prefix=f"layers.{i}.modulelist.0.")
        if i % 2 == 1:
            tok = torch.roll(tok.reshape(1, 8, 8, -1), (2, 2), (1, 2)).reshape(1, 64, -1)
    want = oracle.output_stage(cfg, sd, tok, t)
    torch.testing.assert_close(got, want, rtol=1e-5, atol=1e-5)


def test_sigma_schedule_closed_form():
    t = oracle.sigma_schedule(10, 0.2, 500.0, 1.0)
    assert t.shape == (11,) and t[-1] == 0
    assert abs(t[0].item() - math.atan(500.0)) < 1e-5
    assert abs(t[9].item() - math.atan(0.2)) < 1e-6
    mid = (500 ** 0.1 + (4 / 9) * (0.2 ** 0.1 - 500 ** 0.1)) ** 10
    assert abs(t[4].item() - math.atan(mid)) < 1e-5
    assert (t[:-1] > t[1:]).all()


def test_sampler_closed_forms():
    ts = oracle.sigma_schedule(6).double()
    cond, lat = torch.zeros(1, 3, 2, dtype=torch.float64), torch.randn(1, 3, 2, dtype=torch.float64)
    # F == 0  =>  x_N = sigma_d * latents
    out = oracle.sample(lambda m, t: torch.zeros_like(m[..., :2]), cond, lat, ts, sigma_data=2.0)
    torch.testing.assert_close(out, 2.0 * lat)
    # linear field F = a * x / sigma_d  =>  Heun factor (1 + a D + (a D)^2 / 2) per step, Euler (1 + a D) on the last
    a, sd_ = 0.3, 1.5
    out = oracle.sample(lambda m, t: a * m[..., :2], cond, lat, ts, sigma_data=sd_)
    fac = 1.0
    for i in range(6):
        D = (ts[i + 1] - ts[i]).item()
        fac *= (1 + a * D + 0.5 * (a * D) ** 2) if i < 5 else (1 + a * D)
    torch.testing.assert_close(out, sd_ * lat * fac, rtol=1e-10, atol=1e-12)
    # the denoiser sees [x / sigma_d | cond] and the current noise level
    seen = []
    oracle.sample(lambda m, t: (seen.append((m.shape[-1], float(t))), torch.zeros_like(m[..., :2]))[1],
                  torch.ones(1, 3, 5, dtype=torch.float64), lat, ts)
    assert len(seen) == 2 * 6 - 1 and all(c == 7 for c, _ in seen)
    assert abs(seen[0][1] - ts[0].item()) < 1e-12 and abs(seen[1][1] - ts[1].item()) < 1e-12


def test_rollout_feedback():
    g = torch.Generator().manual_seed(1)
    state0 = torch.randn(1, 4, 3)
    xm, xs, tm, tsd = torch.tensor([1., 2., 3.]), torch.tensor([2., 2., 4.]), torch.tensor([.1, .2, .3]), torch.tensor([.5, .5, .5])
    states = oracle.rollout(lambda m, t: torch.zeros_like(m[..., :3]), state0, 2, 3, g, x_mean=xm, x_std=xs, t_mean=tm, t_std=tsd)
    # F == 0 => each sample equals its latents; replay the feedback by hand
    g2 = torch.Generator().manual_seed(1)
    X = state0 * xs + xm
    for k in range(2):
        y = torch.randn(state0.shape, generator=g2)
        X = X + (y * tsd + tm)
        torch.testing.assert_close(states[k], (X - xm) / xs)


def test_rollout_conditioning_order_and_step_indexing():
    """Known answer for the per-step conditioning of inference.py:133, cat([state, rad_T[k], gp, lsm, rad_T[k+1]]): a
    probe denoiser that returns one input channel makes F constant in x, so the sampler's result is
    x_N = sigma_d * (latents + (t_N - t_0) * F) = sigma_d * (latents - t_0 * F) whatever the number of Heun steps;
    reading a different channel per probe shows which tensor (and which forecast step's slice) sits where."""
    B, S, C, Cf, Cs, Ce, n_fc, n_diff, sd_ = 2, 5, 3, 2, 2, 1, 3, 4, 1.5
    g = torch.Generator().manual_seed(2)
    state0 = torch.randn(B, S, C, generator=g, dtype=torch.float64)
    forcing = torch.randn(n_fc + 1, 1, S, Cf, generator=g, dtype=torch.float64)  # one batch entry: broadcast over members
    static = torch.randn(B, S, Cs, generator=g, dtype=torch.float64)
    extra = torch.randn(n_fc, B, S, Ce, generator=g, dtype=torch.float64)
    lat = torch.randn(n_fc, B, S, C, generator=g, dtype=torch.float64)
    t0 = oracle.sigma_schedule(n_diff, sigma_data=sd_)[0].double()
    # channel layout the denoiser sees: [x / sigma_d (C) | state (C) | forcing[k] (Cf) | static (Cs) | forcing[k+1] (Cf) | extra[k] (Ce)]
    off_state, off_f0, off_st, off_f1, off_ex = C, 2 * C, 2 * C + Cf, 2 * C + Cf + Cs, 2 * C + 2 * Cf + Cs
    probes = {
        "forcing[k]": (off_f0 + 1, lambda k: forcing[k, :, :, 1].expand(B, S)),
        "static": (off_st, lambda k: static[:, :, 0]),
        "forcing[k+1]": (off_f1, lambda k: forcing[k + 1, :, :, 0].expand(B, S)),
        "extra[k]": (off_ex, lambda k: extra[k, :, :, 0]),
    }
    for name, (ch, want_fn) in probes.items():
        seen_width = []

        def den(m, t, ch=ch):
            seen_width.append(m.shape[-1])
            return m[..., ch:ch + 1].expand(-1, -1, C)

        states = oracle.rollout(den, state0, n_fc, n_diff, sigma_data=sd_, forcing=forcing, static=static, extra_cond=extra,
                                latents=lat)
        assert set(seen_width) == {2 * C + 2 * Cf + Cs + Ce}
        X = state0.clone()
        for k in range(n_fc):
            X = X + sd_ * (lat[k] - t0 * want_fn(k).unsqueeze(-1))
            torch.testing.assert_close(states[k], X, rtol=1e-5, atol=1e-5, msg=name)
    # the state itself is the first conditioning block, and it is the fed-back one from the second step on
    states = oracle.rollout(lambda m, t: m[..., off_state:off_state + C], state0, 2, n_diff, sigma_data=sd_, forcing=forcing,
                            static=static, latents=lat[:2])
    X1 = state0 + sd_ * (lat[0] - t0 * state0)
    X2 = X1 + sd_ * (lat[1] - t0 * X1)
    torch.testing.assert_close(states[0], X1, rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(states[1], X2, rtol=1e-5, atol=1e-5)
