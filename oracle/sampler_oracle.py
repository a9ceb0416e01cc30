"""TrigFlow ODE sampler and autoregressive rollout, CPU restatement.  TEST INFRASTRUCTURE ONLY.

Follows src/aeris_wp_inference/inference.py:76-82 (noise schedule) and :132-186 (Heun loop and
autoregressive feedback).  ``denoiser(model_in, t)`` is any callable mapping
``[B, S, C_state + C_cond]`` and a noise level ``t[1]`` to ``[B, S, C_state]``.
"""
from __future__ import annotations

import torch


def sigma_schedule(n_steps, sigma_min=0.2, sigma_max=500.0, sigma_data=1.0, rho=10, dtype=torch.float32):
    """t_i = atan(sigma_i / sigma_data), sigma_i on the rho-ramp, with a final 0 appended."""
    ramp = torch.linspace(0, 1, n_steps, dtype=dtype)
    lo, hi = sigma_min ** (1 / rho), sigma_max ** (1 / rho)
    sig = (hi + ramp * (lo - hi)) ** rho
    t = torch.atan(sig / sigma_data)
    return torch.cat([t, torch.zeros_like(t[:1])])


def sample(denoiser, cond, latents, t_steps, sigma_data=1.0):
    """Second-order Heun on dx/dt = sigma_d * F(x/sigma_d, cond, t); Euler on the last step.

    inference.py:134-178.  ``cond`` is concatenated AFTER the state channels (inference.py:160).
    """
    n = t_steps.numel() - 1
    x = latents * sigma_data
    for i in range(n):
        s, t = t_steps[i], t_steps[i + 1]
        delta = t - s
        F_s = denoiser(torch.cat([x / sigma_data, cond], dim=2), s.view(1))
        x_euler = x + delta * sigma_data * F_s
        if i < n - 1:
            F_t = denoiser(torch.cat([x_euler / sigma_data, cond], dim=2), t.view(1))
            x = x + delta * sigma_data * 0.5 * (F_s + F_t)
        else:
            x = x_euler
    return x


def rollout(denoiser, state0, n_forecast, n_diffusion, generator=None, sigma_min=0.2, sigma_max=500.0,
            sigma_data=1.0, x_mean=None, x_std=None, t_mean=None, t_std=None, forcing=None, static=None,
            extra_cond=None, latents=None):
    """Autoregressive forecast (inference.py:127-186).

    Per forecast step k the conditioning is ``cat([state, forcing[k], static, forcing[k+1], extra])`` along the
    channels (inference.py:133: ``cat([condition, rad_T[k], gp, lsm, rad_T[k+1]])`` with forcing = rad_T and
    static = cat([gp, lsm])); then ``X <- X + unstandardize_t(sample)`` and ``state <- standardize_x(X)``
    (inference.py:180-186; era5.py:95-114: standardise = (x - mean) / std, un-standardise = x * std + mean).
    ``state0`` is the standardised state ``[B, S, C]``; means / stds default to 0 / 1; ``forcing``
    ``[n_forecast + 1, 1|B, S, Cf]``; ``static`` ``[1|B, S, Cs]``; ``extra_cond`` ``[1|B, S, Ce]`` or one per step
    ``[n_forecast, 1|B, S, Ce]``; ``latents`` ``[n_forecast, B, S, C]`` replaces the draws from ``generator``.
    Returns the list of standardised states after every forecast step.
    """
    B, _, C = state0.shape
    one, zero = torch.ones(C), torch.zeros(C)
    x_mean = zero if x_mean is None else x_mean
    t_mean = zero if t_mean is None else t_mean
    x_std = one if x_std is None else x_std
    t_std = one if t_std is None else t_std
    t_steps = sigma_schedule(n_diffusion, sigma_min, sigma_max, sigma_data)

    def bcast(t):
        return t.expand(B, *t.shape[1:])

    cond = state0.clone()
    X_un = state0 * x_std + x_mean
    states = []
    for k in range(n_forecast):
        parts = [cond]
        if forcing is not None:
            parts.append(bcast(forcing[k]))
        if static is not None:
            parts.append(bcast(static))
        if forcing is not None:
            parts.append(bcast(forcing[k + 1]))
        if extra_cond is not None:
            parts.append(bcast(extra_cond if extra_cond.dim() == 3 else extra_cond[k]))
        c = torch.cat(parts, dim=2)
        lat = latents[k] if latents is not None else torch.randn(state0.shape, generator=generator)
        y = sample(denoiser, c, lat, t_steps, sigma_data)
        X_un = X_un + (y * t_std + t_mean)
        cond = (X_un - x_mean) / x_std
        states.append(cond.clone())
    return states
