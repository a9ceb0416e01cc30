"""TrigFlow ODE sampler (second-order Heun) and autoregressive rollout around the denoiser.

Mirrors ``rollout()`` of src/aeris_wp_inference/inference.py (noise schedule :76-82, Heun loop
:132-178, autoregressive feedback :180-186) with everything resident on the device: the noise
levels live in a device tensor, there is no host synchronisation and no printing inside the loop,
so the whole forecast step can be captured into a HIP graph.
"""
from __future__ import annotations

from typing import Optional

import torch


def sigma_schedule(n_steps, sigma_min=0.2, sigma_max=500.0, sigma_data=1.0, rho=10, device="cpu"):
    """t_i = atan(sigma_i / sigma_data) on the rho-ramp, final 0 appended  (inference.py:76-82)."""
    ramp = torch.linspace(0, 1, n_steps, dtype=torch.float32, device=device)
    lo, hi = sigma_min ** (1 / rho), sigma_max ** (1 / rho)
    sig = (hi + ramp * (lo - hi)) ** rho
    t = torch.atan(sig / sigma_data)
    return torch.cat([t, torch.zeros_like(t[:1])])


class TrigFlowSampler:
    def __init__(self, model, n_steps=10, sigma_min=0.2, sigma_max=500.0, sigma_data=1.0, device="cuda"):
        self.model = model
        self.n_steps = n_steps
        self.sigma_data = float(sigma_data)
        self.t_steps = sigma_schedule(n_steps, sigma_min, sigma_max, sigma_data, device=device)
        self._graph = None

    def _denoise(self, x, cond, t):
        # the condition channels follow the state channels (inference.py:160); the division by sigma_data and the
        # concatenation happen inside the embedding's operand preparation
        return self.model(x, t, cond=cond, x_div=self.sigma_data)

    @torch.no_grad()
    def sample(self, cond: torch.Tensor, latents: torch.Tensor) -> torch.Tensor:
        """cond [B, S, C_cond], latents [B, S, C] ~ N(0,1) -> sample [B, S, C]; 2*n_steps-1 denoiser calls."""
        sd, ts, n = self.sigma_data, self.t_steps, self.n_steps
        x = latents * sd
        for i in range(n):
            s, t = ts[i:i + 1], ts[i + 1:i + 2]
            step = (t - s) * sd
            F_s = self._denoise(x, cond, s)
            x_euler = x + step * F_s
            if i < n - 1:
                F_t = self._denoise(x_euler, cond, t)
                x = x + (0.5 * step) * (F_s + F_t)
            else:
                x = x_euler
        return x

    # ---- HIP-graph replay of one forecast step -------------------------------------------------
    def capture(self, cond_example: torch.Tensor, latents_example: torch.Tensor, warmup: int = 1):
        """Capture ``sample`` into a HIP graph with static input/output buffers."""
        self._cond = cond_example.clone()
        self._lat = latents_example.clone()
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(warmup):
                self.sample(self._cond, self._lat)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        torch.cuda.empty_cache()  # the warm-up's cached blocks would sit next to the graph's own pool
        self._graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(self._graph):
            self._out = self.sample(self._cond, self._lat)
        return self

    def sample_graph(self, cond: torch.Tensor, latents: torch.Tensor) -> torch.Tensor:
        if self._graph is None:
            raise RuntimeError("call capture() first")
        self._cond.copy_(cond)
        self._lat.copy_(latents)
        self._graph.replay()
        return self._out

    @torch.no_grad()
    def rollout(self, state0: torch.Tensor, n_forecast: int, generator: Optional[torch.Generator] = None,
                x_mean=None, x_std=None, t_mean=None, t_std=None, extra_cond=None, use_graph=False):
        """Autoregressive forecast (inference.py:127-186): X <- X + unstd_t(sample), cond <- std_x(X).

        ``state0`` is the standardised state [B, S, C]; means / stds are per-channel tensors [C] on the
        device (identity when omitted).  Returns the standardised state after every forecast step.
        """
        dev = state0.device
        C = state0.shape[-1]
        one, zero = torch.ones(C, device=dev), torch.zeros(C, device=dev)
        x_mean = zero if x_mean is None else x_mean
        t_mean = zero if t_mean is None else t_mean
        x_std = one if x_std is None else x_std
        t_std = one if t_std is None else t_std
        cond = state0.clone()
        X_un = state0 * x_std + x_mean
        states = []
        for _ in range(n_forecast):
            c = cond if extra_cond is None else torch.cat([cond, extra_cond], dim=2)
            lat = torch.randn(state0.shape, generator=generator, device=dev)
            y = self.sample_graph(c, lat) if use_graph else self.sample(c, lat)
            X_un = X_un + (y * t_std + t_mean)
            cond = (X_un - x_mean) / x_std
            states.append(cond.clone())
        return states
