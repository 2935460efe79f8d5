#!/usr/bin/env python3
"""Writes tests/golden/w4a4_emulated_257x128x128.npz.

The reference ships no golden vectors and its CUDA kernel cannot run here, so
this fixture is produced by the lane-by-lane emulation of the reference's
kernels in tests/ptx_emulation.py (CUDA packers with ldmatrix semantics,
mma.m16n8k64 fragments, scale broadcasts, staged store) on one seeded input:
fp16 X [257, 128] and W [128, 128] ~ N(0,1), channel scales absmax/7, fp16
bias, clip 0.95 -- the reference kernel smoke test's recipe at a size the
emulation finishes in seconds.  The arrays are what the reference's entry
points would return: v1 qweight / packed scales (pack_weight_with_scale), v1
qact / ascales / act_scales (quantize_activation_per_token), the int32
accumulators and the fp16 output (linear_vdm_w4a4).

Run from the repository root:  python tests/golden/make_w4a4_fixture.py
"""
import sys
from pathlib import Path

import numpy as np

ROOT = Path(__file__).resolve().parents[2]
sys.path.insert(0, str(ROOT))
from tests import ptx_emulation as E  # noqa: E402


def main():
    M, N, K, clip = 257, 128, 128, 0.95
    rng = np.random.default_rng(20240607)
    x = rng.standard_normal((M, K)).astype(np.float16)
    x[:, 5] *= np.float16(20.0)  # one outlier channel
    x[3] = 0  # an all-zero token
    w = rng.standard_normal((N, K)).astype(np.float16)
    wscale = (np.abs(w.astype(np.float32)).max(axis=1) / 7).astype(np.float16)
    bias = rng.standard_normal(N).astype(np.float16)
    act_scales = E.token_scale_kernel(x, clip)
    qact, ascales = E.act_quantize_per_token_kernel(x, act_scales)
    qweight, wscales_packed = E.weight_quantize_per_channel_kernel(w, wscale)
    y, acc = E.linear_w4a4_kernel(qact, qweight, ascales, wscales_packed, bias, M, N, K, return_acc=True)
    out = Path(__file__).with_name("w4a4_emulated_257x128x128.npz")
    np.savez_compressed(out, x=x, w=w, wscale=wscale, bias=bias, clip=np.float32(clip), act_scales=act_scales, qact=qact,
                        ascales=ascales, qweight=qweight, wscales_packed=wscales_packed, acc=acc.astype(np.int32), y=y)
    print("wrote", out, out.stat().st_size, "bytes")


if __name__ == "__main__":
    main()
