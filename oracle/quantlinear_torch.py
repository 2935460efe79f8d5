"""Torch restatement of the reference's QuantLinear floating-point path --
TEST/BASELINE INFRASTRUCTURE ONLY (the CPU baseline the benchmark reports).

Follows vdm_infer/quantization/quant_linear.py of the reference:
  * UniformQuantizer.init_qparams (:43-62): symmetric scale =
    max(|min|, |max|) * clip(1.0), clamped at 1e-5, / 7, cast to x.dtype;
    rows = reshape(x.shape[0], -1) ("per_channel", which is per token for a
    2-D activation);
  * UniformQuantizer.quant / dequant (:64-74): clamp(round(x / scale), -8, 7) * scale,
    evaluated in x.dtype;
  * QuantLinear.forward (:173-178): the weight is fake-quantized on EVERY call,
    then the activation, then F.linear(x, w, bias).
The activation scale is frozen after the first call in the reference (:77-78);
`dynamic=True` recomputes it per call, which is what the kernel path does.
"""
from __future__ import annotations

import torch
import torch.nn.functional as F


def sym_scale(x: torch.Tensor, clip: float = 1.0) -> torch.Tensor:
    rows = x.float().reshape(x.shape[0], -1)
    lo = rows.amin(dim=-1, keepdim=True) * clip
    hi = rows.amax(dim=-1, keepdim=True) * clip
    return (torch.maximum(lo.abs(), hi.abs()).clamp(min=1e-5) / 7).to(x.dtype)


def fake_quant(x: torch.Tensor, scale: torch.Tensor) -> torch.Tensor:
    rows = x.reshape(x.shape[0], -1)
    return (torch.clamp(torch.round(rows / scale), -8, 7) * scale).reshape(x.shape)


class QuantLinearTorchPath:
    def __init__(self, weight: torch.Tensor, bias, dynamic: bool = True):
        self.weight, self.bias, self.dynamic = weight, bias, dynamic
        self.wscale = sym_scale(weight)
        self.ascale = None

    def __call__(self, x: torch.Tensor) -> torch.Tensor:
        w = fake_quant(self.weight, self.wscale)  # per forward, as the reference does
        if self.dynamic or self.ascale is None:
            self.ascale = sym_scale(x)
        return F.linear(fake_quant(x, self.ascale), w, self.bias)
