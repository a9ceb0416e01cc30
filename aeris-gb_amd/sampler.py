"""TrigFlow ODE sampler (second-order Heun) and autoregressive rollout around the denoiser.

Mirrors ``rollout()`` of src/aeris_wp_inference/inference.py (noise schedule :76-82, conditioning :133, Heun loop
:136-178, autoregressive feedback :180-186) with everything resident on the device: the noise levels, the
forecast-step counter, the forcings of every step and the state live in device tensors, there is no host
synchronisation and no printing inside the loop, so one whole forecast step - conditioning, latent draw, 2n-1
denoiser calls, un-standardise, accumulate, re-standardise - is one HIP graph that is replayed per step.
"""
from __future__ import annotations

from typing import Optional

import torch

from . import _lib as L


def sigma_schedule(n_steps, sigma_min=0.2, sigma_max=500.0, sigma_data=1.0, rho=10, device="cpu"):
    """t_i = atan(sigma_i / sigma_data) on the rho-ramp, final 0 appended  (inference.py:76-82)."""
    ramp = torch.linspace(0, 1, n_steps, dtype=torch.float32, device=device)
    lo, hi = sigma_min ** (1 / rho), sigma_max ** (1 / rho)
    sig = (hi + ramp * (lo - hi)) ** rho
    t = torch.atan(sig / sigma_data)
    return torch.cat([t, torch.zeros_like(t[:1])])


class _Rollout:
    """Device-resident state of one autoregressive rollout: everything a forecast step reads or writes."""

    def __init__(self, state0, n_forecast, x_mean, x_std, t_mean, t_std, forcing, static, extra_cond, latents):
        dev, C = state0.device, state0.shape[-1]
        B = state0.shape[0]

        def vec(v, fill):
            return torch.full((C,), fill, device=dev) if v is None else v.to(dev, torch.float32).reshape(C).clone()

        self.x_mean, self.x_std, self.t_mean, self.t_std = vec(x_mean, 0.0), vec(x_std, 1.0), vec(t_mean, 0.0), vec(t_std, 1.0)
        self._cond0 = state0.to(torch.float32).clone()
        self.cond = self._cond0.clone()  # standardised state, the first C conditioning channels
        self.x_un = torch.empty_like(self.cond)  # un-standardised state (inference.py:117), set by reset()
        self.k = torch.zeros(1, dtype=torch.long, device=dev)  # forecast step, advanced on the device
        self.n_forecast = n_forecast
        self.states = torch.empty((n_forecast,) + tuple(state0.shape), dtype=torch.float32, device=dev)

        def per_batch(t, name):
            if t.shape[-3] not in (1, B):
                raise ValueError(f"{name}: batch {t.shape[-3]} is neither 1 nor {B}")
            return t.to(dev, torch.float32).contiguous()

        self.forcing = None
        if forcing is not None:  # [n_forecast + 1, 1|B, S, Cf]: rad_T of inference.py:133
            if forcing.dim() != 4 or forcing.shape[0] < n_forecast + 1:
                raise ValueError(f"forcing must be [>= {n_forecast + 1}, 1|B, S, Cf], got {tuple(forcing.shape)}")
            self.forcing = per_batch(forcing, "forcing")
        self.static = None if static is None else per_batch(static, "static")
        self.extra = None
        if extra_cond is not None:  # [1|B, S, Ce] the same for every step, or [n_forecast, 1|B, S, Ce] one per step
            self.extra = per_batch(extra_cond, "extra_cond")
            if self.extra.dim() == 4 and self.extra.shape[0] < n_forecast:
                raise ValueError("extra_cond has fewer entries than forecast steps")
        self.latents = None
        if latents is not None:
            if tuple(latents.shape) != (n_forecast,) + tuple(state0.shape):
                raise ValueError(f"latents must be [{n_forecast}, *state0.shape]")
            self.latents = latents.to(dev, torch.float32).contiguous()
        self.B = B
        self.graph, self.step = None, None
        self.steps_per_replay = 1  # forecast steps recorded in ``graph``
        self._done = 0
        self.reset()

    def reset(self):
        """Back to the initial state and forecast step 0 (device-side copies; no synchronisation)."""
        self.cond.copy_(self._cond0)
        torch.addcmul(self.x_mean, self.cond, self.x_std, out=self.x_un)
        self.k.zero_()
        self._done = 0  # host-side mirror of k: the device-side indexing is never asked for a step that does not exist

    def run(self, n: Optional[int] = None):
        """Advance by ``n`` forecast steps (default: all that remain) -> the states tensor [n_forecast, B, S, C]."""
        n = self.n_forecast - self._done if n is None else n
        if n < 0 or self._done + n > self.n_forecast:
            raise ValueError(f"{self._done} of {self.n_forecast} forecast steps are done; cannot run {n} more (reset() first)")
        if self.graph is not None and n % self.steps_per_replay:
            raise ValueError(f"the captured graph holds {self.steps_per_replay} forecast steps; {n} is not a multiple of that")
        self._done += n
        if self.graph is not None:
            for _ in range(n // self.steps_per_replay):
                self.graph.replay()
        else:
            for _ in range(n):
                self.step()
        return self.states

    def _expand(self, t):
        return t if t.shape[0] == self.B else t.expand(self.B, *t.shape[1:])

    def conditioning(self):
        """[state | forcing[k] | static | forcing[k+1] | extra] along the channels (inference.py:133)."""
        parts = [self.cond]
        if self.forcing is not None:
            parts.append(self._expand(self.forcing.index_select(0, self.k)[0]))
        if self.static is not None:
            parts.append(self._expand(self.static))
        if self.forcing is not None:
            parts.append(self._expand(self.forcing.index_select(0, self.k + 1)[0]))
        if self.extra is not None:
            parts.append(self._expand(self.extra if self.extra.dim() == 3 else self.extra.index_select(0, self.k)[0]))
        return parts[0] if len(parts) == 1 else torch.cat(parts, dim=2)


class TrigFlowSampler:
    def __init__(self, model, n_steps=10, sigma_min=0.2, sigma_max=500.0, sigma_data=1.0, device="cuda"):
        L.call("aeris_init")  # kernel attributes are set here, never inside a stream capture
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

    # ---- HIP-graph replay of one sampling pass ---------------------------------------------------
    def capture(self, cond_example: torch.Tensor, latents_example: torch.Tensor, warmup: int = 1):
        """Capture ``sample`` into a HIP graph with static input/output buffers."""
        self._cond = cond_example.clone()
        self._lat = latents_example.clone()
        self._graph = self._capture(lambda: self.sample(self._cond, self._lat), warmup)
        self._out = self._captured
        return self

    @staticmethod
    def _side_stream():
        """A fresh stream for warm-up work, entered only once the current stream has drained.  The block intermediates
        are shared per device and change hands between streams only when their last user has nothing pending
        (ops.workspace); an event wait alone would order the two streams correctly but leave that check to timing."""
        cur = torch.cuda.current_stream()
        cur.synchronize()
        side = torch.cuda.Stream()
        side.wait_stream(cur)
        return side

    def _capture(self, fn, warmup, generator=None):
        side = self._side_stream()
        with torch.cuda.stream(side):
            for _ in range(warmup):
                fn()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        torch.cuda.empty_cache()  # the warm-up's cached blocks would sit next to the graph's own pool
        graph = torch.cuda.CUDAGraph()
        if generator is not None:
            graph.register_generator_state(generator)
        with torch.cuda.graph(graph):
            self._captured = fn()
        return graph

    def sample_graph(self, cond: torch.Tensor, latents: torch.Tensor) -> torch.Tensor:
        if self._graph is None:
            raise RuntimeError("call capture() first")
        self._cond.copy_(cond)
        self._lat.copy_(latents)
        self._graph.replay()
        return self._out

    # ---- autoregressive rollout -------------------------------------------------------------------
    def _forecast_step(self, ro: _Rollout, generator):
        """One forecast step on the rollout state ``ro`` (inference.py:130-186), all on the device."""
        c = ro.conditioning()
        if ro.latents is not None:
            lat = ro.latents.index_select(0, ro.k)[0]
        else:
            lat = torch.randn(ro.cond.shape, generator=generator, device=ro.cond.device)  # inference.py:135
        y = self.sample(c, lat)
        ro.x_un.add_(y * ro.t_std + ro.t_mean)  # X <- X + unstandardize_t(Y)   (inference.py:180-183, era5.py:107-114)
        torch.div(ro.x_un - ro.x_mean, ro.x_std, out=ro.cond)  # standardize_x  (inference.py:186, era5.py:95-99)
        ro.states.index_copy_(0, ro.k, ro.cond.unsqueeze(0))
        ro.k.add_(1)

    @torch.no_grad()
    def begin_rollout(self, state0: torch.Tensor, n_forecast: int, generator: Optional[torch.Generator] = None,
                      x_mean=None, x_std=None, t_mean=None, t_std=None, forcing=None, static=None, extra_cond=None,
                      latents=None, use_graph=False, graph_warmup: int = 0, graph_steps: int = 1) -> "_Rollout":
        """Set up an autoregressive forecast (arguments: see ``rollout``) and, with ``use_graph``, capture
        ``graph_steps`` consecutive forecast steps as one HIP graph (1: the graph is one forecast step and is replayed
        per step; n_forecast: the whole rollout is one graph and one replay), after ``graph_warmup`` eager steps whose
        effect on the state, the step counter and the generator is undone.  The forecast-step counter, the forcings and the state store are indexed on the
        device, so the same recorded step serves every position of the rollout.  ``run()`` of the returned object
        advances it; ``reset()`` puts it back to ``state0`` and step 0."""
        if not 0 <= graph_warmup <= n_forecast:
            raise ValueError(f"graph_warmup must lie in 0..{n_forecast} (the warm-up steps are forecast steps)")
        if graph_steps < 1 or n_forecast % graph_steps:
            raise ValueError(f"graph_steps must divide n_forecast = {n_forecast}")
        ro = _Rollout(state0, n_forecast, x_mean, x_std, t_mean, t_std, forcing, static, extra_cond, latents)
        if use_graph and generator is None and latents is None:
            generator = torch.cuda.default_generators[state0.device.index or 0]
        gen = generator if latents is None else None
        ro.step = lambda: self._forecast_step(ro, gen)
        if use_graph:
            # the default generator is registered with every graph; any other one has to be registered by hand
            own = gen if gen is not None and gen is not torch.cuda.default_generators[state0.device.index or 0] else None
            if graph_warmup:
                # the warm-up steps draw latents like any other step: the generator is put back afterwards, so that a
                # seeded rollout gives the same forecast with and without warm-up, eager or replayed
                rng = gen.get_state() if gen is not None else None
                side = self._side_stream()
                with torch.cuda.stream(side):
                    for _ in range(graph_warmup):
                        ro.step()
                torch.cuda.current_stream().wait_stream(side)
                side.synchronize()
                if rng is not None:
                    gen.set_state(rng)
                ro.reset()

            def steps():
                for _ in range(graph_steps):
                    ro.step()

            ro.steps_per_replay = graph_steps
            ro.graph = self._capture(steps if graph_steps > 1 else ro.step, 0, generator=own)
            ro.reset()
        return ro

    @torch.no_grad()
    def rollout(self, state0: torch.Tensor, n_forecast: int, generator: Optional[torch.Generator] = None, **kw):
        """Autoregressive forecast (inference.py:127-186): per step the conditioning is
        ``cat([state, forcing[k], static, forcing[k+1], extra_cond])`` (inference.py:133 with forcing = rad_T and
        static = cat([gp, lsm])), then X <- X + unstd_t(sample), state <- std_x(X).

        ``state0`` is the standardised state [B, S, C]; ``x_mean, x_std, t_mean, t_std`` are per-channel tensors [C]
        (identity when omitted); ``forcing`` [n_forecast + 1, 1|B, S, Cf]; ``static`` [1|B, S, Cs]; ``extra_cond``
        [1|B, S, Ce] or one per step [n_forecast, 1|B, S, Ce]; ``latents`` [n_forecast, B, S, C] replaces the draw
        from ``generator``.  ``use_graph``: the forecast step is captured once and replayed n_forecast times
        (``graph_steps=n_forecast``: the whole rollout is captured as one graph and replayed once).
        Returns the standardised state after every forecast step, [n_forecast, B, S, C].
        """
        ro = self.begin_rollout(state0, n_forecast, generator, **kw)
        self._last_rollout = ro  # a captured graph's memory pool has to outlive the replays still in flight
        return ro.run()
