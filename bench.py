"""Benchmark of the hot path: one full denoiser step on the 720x1440 grid, bf16, one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload config3|config2|config1] [--no-cpu-baseline]

A "step" is one denoiser forward (one function evaluation of the diffusion sampler): 138-channel input ->
1x1 embedding to dim 1536 -> 24 Swin blocks (alternating un-shifted / half-window-shifted 16x16 windows,
24 heads x 64, LayerNorm + per-block scale/shift from the noise-level embedding, rel-pos bias, shift mask,
GELU MLP x4) -> linear head to 69 channels.  Random-init weights, Gaussian inputs, all resident in HBM
before the timed region.  Prints ONE JSON line.
"""
from __future__ import annotations

import argparse
import importlib
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2500.0  # MI355X dense bf16 MFMA
PEAK_HBM_GBS = 8000.0      # MI355X HBM3E
# Bytes that crossed the L2 <-> fabric boundary per launch at the config3 workload (average over the launches of
# one step), from two rocprofv3 --pmc runs (FETCH_SIZE, WRITE_SIZE) scaled by a 1 GiB copy kernel; the summary
# with the commands is profiles/denoiser_step_config3_pmc_traffic.txt.  Not measurable from inside this script.
PMC_TRAFFIC_BYTES = {"config3": {"gemm_256x256_none_f32": 30.169e9 + 6.373e9, "gemm_256x256_none_bf16_plain": 40.273e9 + 9.555e9,
                                 "gemm_256x256_gelu_bf16_plain": 31.556e9 + 12.740e9, "window_attention": 9.573e9 + 3.187e9,
                                 "qkv_window_attention": 31.338e9 + 3.185e9,
                                 "norm_modulate": 6.463e9 + 3.185e9, "output_stage": 6.384e9 + 0.286e9}}

WORKLOADS = {
    # name: grid, dim, heads, head_dim, window, mlp, blocks, in/out channels
    "config3": dict(image_shape=(720, 1440), dim=1536, heads=24, head_dim=64, window=16, mlp_dim=6144, blocks=24,
                    cin=138, cout=69, desc="configs[3]: full denoiser step, 720x1440 grid, 24 blocks, dim 1536, 24x64 heads, 16x16 windows"),
    "config2": dict(image_shape=(720, 1440), dim=1024, heads=16, head_dim=64, window=16, mlp_dim=4096, blocks=1,
                    cin=138, cout=69, desc="configs[2]-shaped denoiser with ONE shifted block, dim 1024, 16x64 heads"),
    "config4": dict(image_shape=(720, 1440), dim=1536, heads=24, head_dim=64, window=16, mlp_dim=6144, blocks=24,
                    cin=138, cout=69, rollout=True,
                    desc="configs[4]: ensemble rollout with the configs[3] denoiser, members as batch, Heun ODE sampler "
                         "replayed as one HIP graph per forecast step"),
    "refwin": dict(image_shape=(720, 1440), dim=1536, heads=12, head_dim=128, window=60, mlp_dim=6144, blocks=24,
                   cin=138, cout=69, preset="ref",
                   desc="configs[3] grid and widths with the reference's own block (model.py: RMSNorm, 3-way modulation before "
                        "the norm, SwiGLU, no biases) and window geometry (60x60 windows of 3600 tokens, 12 heads x 128)"),
    "config1": dict(image_shape=(180, 360), dim=512, heads=8, head_dim=64, window=12, mlp_dim=2048, blocks=2,
                    cin=138, cout=69, desc="configs[1]-shaped denoiser, 180x360 grid, 2 blocks, dim 512, 12x12 windows"),
}


def build_model(pkg, torch, wl, device, residual_dtype, init=True):
    ws = wl["window"]
    model = pkg.LocalAERIS(device_mesh=None, heads=wl["heads"], dim=wl["dim"], head_dim=wl["head_dim"],
                           mlp_dim=wl["mlp_dim"], window_size=(ws, ws), image_shape=wl["image_shape"], rope_base=10_000,
                           sublayers=1, sinusoidal_emb_max_period=10_000, n_layers=wl["blocks"] + 2,
                           model_in_channels=wl["cin"], model_out_channels=wl["cout"], residual_dtype=residual_dtype,
                           **(dict(preset="ref") if wl.get("preset") == "ref" else dict(preset="spec", mod_ways=2)))
    model = model.to(device)
    if not init:
        return model
    g = torch.Generator(device=device).manual_seed(0)
    with torch.no_grad():
        for name, p in model.named_parameters():
            if p.dim() >= 2:  # Linear weights and the rel-pos tables: trunc-normal(0.02); effectively un-truncated
                p.copy_((0.02 * torch.randn(p.shape, generator=g, device=device, dtype=torch.float32)).clamp_(-2, 2).to(p.dtype))
            elif name.endswith("bias"):
                p.zero_()
            else:
                p.fill_(1.0)
    return model


def run_rollout(args, pkg, torch, wl, model, dev, res_dt):
    """configs[4]: `--steps` autoregressive forecast steps (a step = one forecast step = 2n-1 denoiser calls on a
    batch of `--ensemble` members), the sampler loop replayed as a HIP graph.  The roofline object is the dominant GEMM
    of one eager denoiser call at this batch.  cpu_baseline and parity are those of one member's denoiser call (the
    oracle on a strip of the grid, as for configs[3]): a member's call is the unit `value` counts, so the CPU rate in
    denoise steps/s carries over unchanged; the line says that it is derived."""
    import threading
    H, W = wl["image_shape"]
    S, B, C = H * W, args.ensemble, wl["cout"]
    done = threading.Event()

    def heartbeat():  # a forecast step is minutes of GPU time with nothing to print; say that the run is alive
        t_start = time.perf_counter()
        while not done.wait(45.0):
            print(f"bench.py: rollout running, {time.perf_counter() - t_start:.0f} s", file=sys.stderr, flush=True)

    threading.Thread(target=heartbeat, daemon=True).start()
    g = torch.Generator(device=dev).manual_seed(1)
    with torch.no_grad():  # per-kernel timing of one eager denoiser call at this batch (also the warm-up)
        x = torch.randn(B, S, wl["cin"], generator=g, device=dev)
        t = torch.rand(B, generator=g, device=dev) * (math.pi / 2)
        model(x, t)
        pkg.ops.profile_begin()
        model(x, t)
        rec = pkg.ops.profile_end()
        del x
    smp = pkg.TrigFlowSampler(model, n_steps=args.sampler_steps, device=dev)
    state0 = torch.randn(B, S, C, generator=g, device=dev)
    nfe = 2 * args.sampler_steps - 1
    # one HIP graph = one whole forecast step: latent draw, 2n-1 denoiser calls, un-standardise + accumulate +
    # re-standardise of the state; captured once, replayed per step
    ro = smp.begin_rollout(state0, max(args.steps, args.warmup, 1), g, use_graph=True, graph_warmup=0)
    ro.run(args.warmup)
    ro.reset()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    states = ro.run(args.steps)[:args.steps]
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    finite = bool(torch.isfinite(states).all())
    done.set()
    agg = {}
    for tag, work, unit, ms in rec:
        a = agg.setdefault(tag, {"launches": 0, "work": 0.0, "ms": 0.0, "unit": unit})
        a["launches"] += 1; a["work"] += work; a["ms"] += ms
    dom_tag = max((t_ for t_ in agg if t_.startswith("gemm_256x256")), key=lambda t_: agg[t_]["ms"])
    dom = agg[dom_tag]
    tfl = dom["work"] / (dom["ms"] * 1e-3) / 1e12
    result = {
        "metric": "denoise steps/s + window-attn MFMA util, 720x1440 grid bf16, 1 GPU",
        "value": B * nfe * args.steps / elapsed, "unit": "denoise steps/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": elapsed / args.steps * 1e3, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "forecast_steps_per_s": args.steps / elapsed,
        "config": {"workload": wl["desc"], "tokens": S, "batch": B, "sampler_steps": args.sampler_steps,
                   "denoiser_calls_per_forecast_step": nfe, "step": "one forecast step",
                   "value_counts": "one denoiser call on one member = one denoise step"},
        "roofline": {"kernel": dom_tag, "bound": "mfma", "achieved": tfl, "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                     "frac": tfl / PEAK_BF16_TFLOPS, "traffic": None, "flop_per_launch": dom["work"] / dom["launches"],
                     "avg_launch_ms": dom["ms"] / dom["launches"]},
        "cpu_baseline": None, "output_finite": finite,
    }
    if not args.no_cpu_baseline:
        base, parity = cpu_baseline_and_parity(pkg, torch, wl, model, args.cpu_rows, dev, res_dt)
        base["sample"] += (f"; derived for the rollout: one forecast step = {nfe} denoiser calls x {B} members = {nfe * B} such "
                           f"forwards = {nfe * B / base['value']:.0f} s of CPU time")
        result["cpu_baseline"], result["parity"] = base, parity
        result["gpu_over_cpu"] = result["value"] / base["value"]
    print(json.dumps(result))


def cpu_baseline_and_parity(pkg, torch, wl, model, rows, dev, residual_dtype):
    """The CPU leg and the parity figure in one: the fp32 oracle (this repository's CPU restatement of the reference
    model) runs the WHOLE denoiser - embedding, every block, head - on a strip of the grid, `rows` latitude rows x full
    longitude, with the benchmarked model's own weights.  Its wall time, scaled by the number of strips in the grid, is
    the CPU baseline (windows never mix tokens of different window rows, so a strip of whole window rows is a
    self-contained model run; with one window row the shifted blocks wrap inside it).  The same strip through the HIP
    model gives relative-L2 and max-abs error of the timed configuration at its full depth."""
    import oracle
    H, W = wl["image_shape"]
    ws = wl["window"]
    threads = torch.get_num_threads()
    ref = wl.get("preset") == "ref"
    mk = oracle.OracleConfig.ref if ref else (lambda **kw: oracle.OracleConfig.spec(mod_ways=2, **kw))
    cfg = mk(dim=wl["dim"], heads=wl["heads"], head_dim=wl["head_dim"], mlp_dim=wl["mlp_dim"], window_size=(ws, ws),
             image_shape=(rows, W), n_layers=wl["blocks"] + 2, in_channels=wl["cin"], out_channels=wl["cout"])
    sd = {k: v.detach().float().cpu() for k, v in model.state_dict().items()}
    strip = build_model(pkg, torch, dict(wl, image_shape=(rows, W)), dev, residual_dtype, init=False)
    strip.load_state_dict(model.state_dict())
    g = torch.Generator().manual_seed(2)
    x = torch.randn(1, rows * W, wl["cin"], generator=g)
    t = torch.rand(1, generator=g) * (math.pi / 2)
    with torch.no_grad():
        got = strip(x.to(dev), t.to(dev)).float().cpu()
        warm = torch.randn(512, 512)
        (warm @ warm).sum().item()  # spin up the thread pool
        import threading
        done = threading.Event()

        def heartbeat():  # the oracle prints nothing for up to minutes (the 60x60-window workload); say that the run is alive
            while not done.wait(45.0):
                print(f"bench.py: CPU oracle running, {time.perf_counter() - t0:.0f} s", file=sys.stderr, flush=True)

        t0 = time.perf_counter()
        threading.Thread(target=heartbeat, daemon=True).start()
        try:
            want = oracle.model_forward(cfg, sd, x, t)
            t_strip = time.perf_counter() - t0
        finally:
            done.set()
    del strip
    diff = (got.double() - want.double())
    parity = {"rel_l2": float(diff.norm() / want.double().norm()), "max_abs": float(diff.abs().max()),
              "ref_rms": float(want.double().pow(2).mean().sqrt()), "tolerance_rel_l2": 1e-2,
              "against": f"fp32 CPU oracle, whole denoiser ({wl['blocks']} blocks) on a {rows}x{W} strip, same weights and inputs"}
    scale = H / rows
    try:
        import psutil
        physical, logical = psutil.cpu_count(logical=False), psutil.cpu_count(logical=True)
    except Exception:
        physical, logical = None, os.cpu_count()
    usable = len(os.sched_getaffinity(0)) if hasattr(os, "sched_getaffinity") else logical
    base = {"value": 1.0 / (t_strip * scale), "unit": "denoise steps/s", "cores": threads, "kind": "port",
            "host_physical_cores": physical, "host_logical_cores": logical, "cores_this_process_may_use": usable,
            "sample": f"fp32 torch oracle, full-depth denoiser forward on a {rows}x{W} strip of the grid: {t_strip:.1f} s on "
                      f"{threads} torch threads, scaled x{scale:.0f} strips (extrapolated)"}
    return base, parity


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=3)
    ap.add_argument("--warmup", type=int, default=1)
    ap.add_argument("--workload", default="config3", choices=sorted(WORKLOADS))
    ap.add_argument("--residual", default="f32", choices=["bf16", "f32"],
                    help="dtype of the residual stream between blocks (f32: within 1e-2 of fp32 at 24 blocks; bf16: not)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--cpu-rows", type=int, default=0,
                    help="latitude rows of the strip the CPU oracle runs (a multiple of the window; default: one window row)")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also launch one plain 1 GiB device-to-device copy (a kernel of known traffic, for scaling "
                         "rocprofv3 FETCH_SIZE / WRITE_SIZE readings)")
    ap.add_argument("--no-fused-compare", action="store_true",
                    help="skip the second timing of the step with to_qkv + window attention as ONE kernel")
    ap.add_argument("--ensemble", type=int, default=4, help="config4: ensemble members (batch)")
    ap.add_argument("--sampler-steps", type=int, default=10, help="config4: sampler steps (2n-1 denoiser calls per forecast step)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs the whole grid on ONE GPU; --gpus N > 1 is not supported "
              "(no collectives, no sharding in this tier)", file=sys.stderr)
        sys.exit(2)

    import torch
    pkg = importlib.import_module("aeris-gb_amd")
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; the HIP path has no CPU fallback", file=sys.stderr)
        sys.exit(3)
    dev = torch.device("cuda:0")
    pkg._lib.call("aeris_init")
    wl = WORKLOADS[args.workload]
    H, W = wl["image_shape"]
    S = H * W
    if args.cpu_rows <= 0:
        args.cpu_rows = wl["window"]
    if args.cpu_rows % wl["window"] or H % args.cpu_rows:
        print("bench.py: --cpu-rows must be a multiple of the window size and divide the grid height", file=sys.stderr)
        sys.exit(2)
    res_dt = torch.bfloat16 if args.residual == "bf16" else torch.float32
    model = build_model(pkg, torch, wl, dev, res_dt)
    g = torch.Generator(device=dev).manual_seed(1)
    x = torch.randn(1, S, wl["cin"], generator=g, device=dev)
    t = (torch.rand(1, generator=g, device=dev) * (math.pi / 2))

    if wl.get("rollout"):
        run_rollout(args, pkg, torch, wl, model, dev, res_dt)
        return

    if args.copy_calibration:
        src = torch.ones(1 << 28, dtype=torch.float32, device=dev)  # 1 GiB read + 1 GiB written
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    with torch.no_grad():
        for _ in range(args.warmup):
            out = model(x, t)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            out = model(x, t)
        torch.cuda.synchronize()
        elapsed = time.perf_counter() - t0
        finite = bool(torch.isfinite(out).all())
        # per-kernel timing with HIP events on the launch stream, over the same K steps
        pkg.ops.profile_begin()
        for _ in range(args.steps):
            model(x, t)
        rec = pkg.ops.profile_end()

        # the same step with to_qkv + window attention as ONE kernel (q, k, v never in HBM) where the block shape allows it:
        # timed beside the default so that the choice of the default is a measurement of this run
        fused_rec, fused_elapsed = None, None
        attn_mods = [m for m in model.modules() if isinstance(m, pkg.model.Attention) and
                     pkg.ops.qkv_attention_supported(wl["dim"], m.heads, m.head_dim, m.window_size, m.image_shape)]
        if not args.no_fused_compare and attn_mods:
            was = [m.fuse_qkv for m in attn_mods]
            for m in attn_mods:
                m.fuse_qkv = not m.fuse_qkv
            try:
                model(x, t)
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                for _ in range(args.steps):
                    model(x, t)
                torch.cuda.synchronize()
                fused_elapsed = time.perf_counter() - t0
                pkg.ops.profile_begin()
                for _ in range(args.steps):
                    model(x, t)
                fused_rec = pkg.ops.profile_end()
            finally:
                for m, v in zip(attn_mods, was):
                    m.fuse_qkv = v

    ms_per_step = elapsed / args.steps * 1e3

    def aggregate(records):
        out = {}
        for tag, work, unit, ms in records:
            a = out.setdefault(tag, {"launches": 0, "work": 0.0, "ms": 0.0, "unit": unit})
            a["launches"] += 1
            a["work"] += work
            a["ms"] += ms
        return out

    agg = aggregate(rec)
    kernels = {}
    for tag, a in agg.items():
        rate = a["work"] / (a["ms"] * 1e-3)
        if a["unit"] == "flop":
            kernels[tag] = {"launches_per_step": a["launches"] // args.steps, "avg_ms": a["ms"] / a["launches"],
                            "ms_per_step": a["ms"] / args.steps, "tflops": rate / 1e12,
                            "frac_mfma_peak": rate / 1e12 / PEAK_BF16_TFLOPS}
        else:
            kernels[tag] = {"launches_per_step": a["launches"] // args.steps, "avg_ms": a["ms"] / a["launches"],
                            "ms_per_step": a["ms"] / args.steps, "gbs": rate / 1e9, "frac_hbm_peak": rate / 1e9 / PEAK_HBM_GBS}
    if "window_attention" in kernels:  # q, k, v in + o out, bf16: 8 * S * inner bytes per launch
        k = kernels["window_attention"]
        byts = 8.0 * S * wl["heads"] * wl["head_dim"]
        k["gbs"] = byts / (k["avg_ms"] * 1e-3) / 1e9
        k["frac_hbm_peak"] = k["gbs"] / PEAK_HBM_GBS
    NAMES = {"gemm_256x256_none_bf16_res": "gemm_bf16_nt_persistent_kernel<0, false, false, true, false> (proj / fc2 GEMMs on a bf16 residual stream: x gate + residual)",
             "gemm_256x256_none_bf16": "gemm_bf16_nt_persistent_kernel<0, false, false, false, false>",
             "gemm_256x256_none_bf16_plain": "gemm_bf16_nt_persistent_kernel<0, false, true, false, false> (qkv GEMM)",
             "gemm_256x256_gelu_bf16_plain": "gemm_bf16_nt_persistent_kernel<1, false, true, false, false> (fc1 GEMM + GELU)",
             "gemm_256x256_none_f32": "gemm_bf16_nt_persistent_kernel<0, true, false, false, true> (proj / fc2 GEMMs on the f32 residual stream: x gate + residual)",
             "gemm_256x256_none_f32_plain": "gemm_bf16_nt_persistent_kernel<0, true, true, false, false> (plain GEMM with f32 output)",
             "input_stage": "input_stage_kernel<5, true> (concatenation, positional encoding and embedding Linear in one pass)",
             "gemm_256x256_swiglu_bf16_plain": "gemm_bf16_nt_persistent_kernel<2, false, true, false, false>"}
    big = [t for t in kernels if t.startswith("gemm_256x256")]
    roofline = None
    if big:
        dom_tag = max(big, key=lambda t: kernels[t]["ms_per_step"])  # the kernel the step spends most time in
        dom, a = kernels[dom_tag], agg[dom_tag]
        roofline = {"kernel": NAMES.get(dom_tag, dom_tag),
                    "bound": "mfma", "achieved": dom["tflops"], "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                    "frac": dom["tflops"] / PEAK_BF16_TFLOPS,
                    "traffic": PMC_TRAFFIC_BYTES.get(args.workload, {}).get(dom_tag),
                    "flop_per_launch": a["work"] / a["launches"], "avg_launch_ms": dom["avg_ms"]}

    result = {
        "metric": "denoise steps/s + window-attn MFMA util, 720x1440 grid bf16, 1 GPU",
        "value": args.steps / elapsed, "unit": "denoise steps/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": wl["desc"], "tokens": S, "batch": 1, "residual_stream": args.residual,
                   "preset": ("ref (RMSNorm, shift/scale/gate modulation before the norm, SwiGLU MLP, no biases, bias table or mask)"
                              if wl.get("preset") == "ref" else
                              "spec (LayerNorm, scale/shift modulation, rel-pos bias, shift mask, GELU MLP, biases)")},
        "roofline": roofline, "kernels": kernels, "output_finite": finite,
    }
    if fused_rec is not None:
        other = aggregate(fused_rec)
        default_fused = "qkv_window_attention" in agg
        both = other if not default_fused else agg      # the run in which the one-kernel form was used
        pair = agg if not default_fused else other      # the run with the to_qkv GEMM and the attention kernel apart
        if "qkv_window_attention" in both:
            a = both["qkv_window_attention"]
            one_ms = a["ms"] / a["launches"]
            tfl = a["work"] / (a["ms"] * 1e-3) / 1e12
            inner = wl["heads"] * wl["head_dim"]
            attn_flop = 4.0 * S * wl["window"] ** 2 * inner
            byts = 2.0 * S * wl["dim"] + 2.0 * S * inner + 2.0 * 3 * inner * wl["dim"]  # y in, o out, the weight once
            two = {}
            for tag in ("gemm_256x256_none_bf16_plain", "window_attention"):
                if tag in pair:
                    two[tag] = pair[tag]["ms"] / pair[tag]["launches"]
            result["qkv_attention_one_kernel"] = {
                "kernel": "qkv_window_attention_kernel<HAS_BIAS> (to_qkv GEMM, q scaling, window attention; q, k, v stay in LDS)",
                "is_default": default_fused, "launches_per_step": a["launches"] // args.steps, "avg_ms": one_ms,
                "tflops": tfl, "frac_mfma_peak": tfl / PEAK_BF16_TFLOPS,
                "attention_part_tflops_beside_separate_gemm_time": None,
                "hbm_bytes_algorithmic": byts, "hbm_gbs_algorithmic": byts / (one_ms * 1e-3) / 1e9,
                "frac_hbm_peak": byts / (one_ms * 1e-3) / 1e9 / PEAK_HBM_GBS,
                "two_kernels_avg_ms": two, "two_kernels_sum_ms": sum(two.values()) if len(two) == 2 else None,
                "ms_per_step_with_one_kernel": (fused_elapsed if not default_fused else elapsed) / args.steps * 1e3,
                "ms_per_step_with_two_kernels": (elapsed if not default_fused else fused_elapsed) / args.steps * 1e3,
            }
            if len(two) == 2:
                rest = one_ms - two["gemm_256x256_none_bf16_plain"]
                if rest > 0:
                    result["qkv_attention_one_kernel"]["attention_part_tflops_beside_separate_gemm_time"] = \
                        attn_flop / (rest * 1e-3) / 1e12
    if not args.no_cpu_baseline:
        result["cpu_baseline"], result["parity"] = cpu_baseline_and_parity(pkg, torch, wl, model, args.cpu_rows, dev, res_dt)
        result["gpu_over_cpu"] = result["value"] / result["cpu_baseline"]["value"]
    print(json.dumps(result))


if __name__ == "__main__":
    main()
