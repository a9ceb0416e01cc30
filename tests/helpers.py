"""Shared helpers of the GPU parity tests: build a product module and load the oracle's fp32 weights into it."""
import dataclasses

import torch

import oracle
from oracle import OracleConfig

BLOCK_FIELDS = ("norm", "mod_order", "mod_ways", "mlp", "bias", "rel_pos_bias", "shift_mask", "eps")


def rel_l2(a, b):
    a, b = a.double().cpu(), b.double().cpu()
    return float((a - b).norm() / b.norm().clamp_min(1e-30))


def max_abs(a, b):
    return float((a.double().cpu() - b.double().cpu()).abs().max())


def block_options(cfg: OracleConfig):
    return {k: getattr(cfg, k) for k in BLOCK_FIELDS}


def make_layer(pkg, cfg: OracleConfig, sd, device, shifted=False):
    """SwinLayer (preset spec so that it shifts on its own) carrying the oracle's weights (cast to bf16)."""
    layer = pkg.SwinLayer(None, cfg.dim, cfg.heads, cfg.head_dim, cfg.mlp_dim, cfg.window_size, cfg.image_shape,
                          shifted, 10_000, preset="spec", **block_options(cfg))
    missing = layer.load_state_dict(sd, strict=True)
    return layer.to(torch.bfloat16).to(device)


def make_model(pkg, cfg: OracleConfig, sd, device, residual_dtype=torch.bfloat16, preset="spec"):
    m = pkg.LocalAERIS(device_mesh=None, heads=cfg.heads, dim=cfg.dim, head_dim=cfg.head_dim, mlp_dim=cfg.mlp_dim,
                       window_size=cfg.window_size, image_shape=cfg.image_shape, rope_base=10_000,
                       sublayers=cfg.sublayers, sinusoidal_emb_max_period=cfg.max_period, n_layers=cfg.n_layers,
                       model_in_channels=cfg.in_channels, model_out_channels=cfg.out_channels, preset=preset,
                       residual_dtype=residual_dtype, **block_options(cfg))
    full = dict(sd)
    full["input_stage.ape.inv_freq"] = m.state_dict()["input_stage.ape.inv_freq"]
    m.load_state_dict(full, strict=True)
    return m.to(device)


def branch_tap(pkg, store):
    """A ``tap`` for ``SwinLayer.forward`` that projects the two intermediates the block shows it (attention output,
    activated hidden) without gate or residual, into ``store["attn"]`` / ``store["mlp"]`` - the un-gated branch outputs
    the oracle returns with ``return_branches=True``."""
    ops = pkg.ops

    def tap(name, t, mods):
        if name == "attn":
            store["attn"] = ops.gemm(t, mods[1].wo.weight, mods[1].wo.bias)
        else:
            ff = mods[3]
            w, b = (ff.w2.weight, None) if hasattr(ff, "w2") else (ff.fc2.weight, ff.fc2.bias)
            store["mlp"] = ops.gemm(t.reshape(-1, t.shape[-1]), w, b)
    return tap
