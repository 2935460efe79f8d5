#!/usr/bin/env python3
"""End-to-end harness: Wan-2.1 1.3B W4A4 DiT denoise steps with random-init
packed weights (the fifth benchmark configuration: 480p, 81 frames, 5 steps), reporting the share of step time spent in
the W4A4 kernels.

Latent [2 (CFG pair), 16, 21, 60, 104] ~ N(0,1): the pipeline runs classifier-free
guidance as two sequential forwards of one 32760-token sequence (cond, then
uncond); text context [2, 512, 4096] ~ N(0,1) (one per branch); 5 steps;
BOUNDARY_RATIO 0.4 with guidance_scale_2 = 1 (CFG-drop below t = 400, which a
5-step schedule never reaches).  Prints ONE JSON line.
"""
from __future__ import annotations

import argparse
import json
import sys
import time
from dataclasses import replace
from pathlib import Path

sys.path.insert(0, str(Path(__file__).resolve().parent))


def measure(torch, steps=5, layers=30, frames=21, height=60, width=104, boundary_ratio=0.4, model_name="1.3B", fuse_ln=False,
            fuse_residual=False, fuse_gelu=False, reuse_context=False, warmup_steps=0):
    """Build the harness model, run ``warmup_steps`` untimed denoise steps (and always one untimed forward), then
    time ``steps`` denoise steps; returns the result dict."""
    from dsaquant_amd import wan_harness as W
    from dsaquant_amd.kernels import vdm_w4a4 as v
    from dsaquant_amd.quantization.quant_linear import QuantLinear

    assert v.is_available(), v.load_error()
    dev = "cuda:0"
    torch.cuda.set_device(0)
    base = W.WAN21_1P3B if model_name == "1.3B" else W.WAN21_14B
    wargs = replace(base, num_layers=layers)
    t0 = time.perf_counter()
    model = W.build_quantized(wargs, dev, seed=0)
    build_s = time.perf_counter() - t0
    saved = (W.FeedForward.fuse_gelu, W.Block.fuse_ln, W.Block.fuse_residual, W.WanDiT.reuse_context, W.Attention.cache_cross_kv)
    W.FeedForward.fuse_gelu = bool(fuse_gelu)
    W.Block.fuse_ln = bool(fuse_ln)
    W.Block.fuse_residual = bool(fuse_residual)
    W.WanDiT.reuse_context = W.Attention.cache_cross_kv = bool(reuse_context)
    try:
        n_quant = sum(isinstance(m, QuantLinear) for m in model.modules())
        n_fused = sum(isinstance(m, W.Attention) and m.use_fused_qkv_kernel for m in model.modules())

        g = torch.Generator(device=dev).manual_seed(0)
        latents = torch.randn((2, wargs.in_channels, frames, height, width), generator=g, device=dev)
        context = torch.randn((2, 512, wargs.text_dim), generator=g, device=dev).half()
        tokens = frames * (height // 2) * (width // 2)
        ts = W.unipc_timesteps(steps)

        # warm-up: one forward (the first use of every kernel variant), then whole steps if asked for
        with torch.no_grad():
            model(latents[:1].half(), torch.tensor([ts[0]], device=dev), context[:1])
        if warmup_steps:
            W.denoise(model, latents[:1], context[:1], context[1:], ts[:warmup_steps], boundary_ratio=boundary_ratio)
        torch.cuda.synchronize()

        timers = W.KernelTimers()
        with W.time_w4a4_calls(timers):
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            out, forwards = W.denoise(model, latents[:1], context[:1], context[1:], ts, boundary_ratio=boundary_ratio, timers=timers)
            torch.cuda.synchronize()
            wall = time.perf_counter() - t0
        tot = timers.collect()
        cnt = timers.counts()
        assert torch.isfinite(out).all()
    finally:
        W.FeedForward.fuse_gelu, W.Block.fuse_ln, W.Block.fuse_residual, W.WanDiT.reuse_context, W.Attention.cache_cross_kv = saved
    return {
        "metric": "share of denoise-step time in the W4A4 kernels, Wan-2.1 %s DiT, %d steps" % (model_name, steps),
        "value": round(tot.get("w4a4", 0.0) / (wall * 1e3), 4), "unit": "fraction of wall time",
        "attention_share": round(tot.get("attention", 0.0) / (wall * 1e3), 4),
        "ms_per_step": round(wall * 1e3 / steps, 2), "ms_per_forward": round(wall * 1e3 / forwards, 2), "forwards": forwards,
        "w4a4_ms_per_forward": round(tot.get("w4a4", 0.0) / forwards, 2), "attention_ms_per_forward": round(tot.get("attention", 0.0) / forwards, 2),
        "w4a4_calls_per_forward": cnt.get("w4a4", 0) // forwards, "attention_calls_per_forward": cnt.get("attention", 0) // forwards,
        "tokens_per_forward": tokens, "timesteps": ts, "quant_linears": n_quant, "fused_attention_modules": n_fused,
        "layers": layers, "fuse_gelu": bool(fuse_gelu), "fuse_ln": bool(fuse_ln), "fuse_residual": bool(fuse_residual),
        "reuse_context": bool(reuse_context), "build_s": round(build_s, 1), "data": "synthetic", "n_gpus": 1,
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--steps", type=int, default=5)
    ap.add_argument("--warmup-steps", type=int, default=0)
    ap.add_argument("--layers", type=int, default=30)
    ap.add_argument("--frames", type=int, default=21)
    ap.add_argument("--height", type=int, default=60)
    ap.add_argument("--width", type=int, default=104)
    ap.add_argument("--boundary-ratio", type=float, default=0.4)
    ap.add_argument("--model", default="1.3B", choices=["1.3B", "14B"])
    ap.add_argument("--fuse-ln", action="store_true", help="run the blocks' LayerNorm + modulation inside the following activation quantizers")
    ap.add_argument("--fuse-residual", action="store_true", help="run the blocks' gated residual updates in the preceding GEMM epilogues")
    ap.add_argument("--fuse-gelu", action="store_true", help="evaluate the FFN's GELU inside the second linear's activation quantizer")
    ap.add_argument("--reuse-context", action="store_true",
                    help="embed each context once, keep the cross-attention K/V per prompt, quantize a context once per forward")
    args = ap.parse_args()

    import torch

    print(json.dumps(measure(torch, steps=args.steps, layers=args.layers, frames=args.frames, height=args.height, width=args.width,
                             boundary_ratio=args.boundary_ratio, model_name=args.model, fuse_ln=args.fuse_ln, fuse_residual=args.fuse_residual,
                             fuse_gelu=args.fuse_gelu, reuse_context=args.reuse_context, warmup_steps=args.warmup_steps)))


if __name__ == "__main__":
    main()
