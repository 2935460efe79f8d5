"""Producer fusions around the W4A4 linear that the reference runs as separate
kernels.  They are additions next to the drop-in API (the reference's
``QuantLinear.forward`` has no hook for them), for callers that own the module
code between two linears.

``linear_gelu_vdm_w4a4(x, ...)`` computes ``linear_vdm_w4a4(gelu_tanh(x), ...)``:
the second FFN linear of a Wan block applied to the *pre-activation* output of
the first (FeedForward with activation_fn="gelu-approximate",
vdm_infer/models/wan_vdm/modules/dit_block.py:56 of the reference).  The GELU is
evaluated inside the activation quantizer, so the GELU kernel, its [M, ffn]
fp16 write and the quantizer's re-read of it disappear.
"""
from __future__ import annotations

from typing import Optional

import torch

from . import _lib
from .kernels import vdm_w4a4 as _k


def gelu_tanh(x: torch.Tensor) -> torch.Tensor:
    """fp16 GELU (tanh approximation) with the arithmetic of the fused quantizer:
    fp32 evaluation, one rounding to fp16."""
    lib = _k._load_ext()
    xh = x.half().contiguous()
    _k._check_device_tensor(xh, "input", torch.float16)
    n = xh.numel()
    if n % 2:
        raise ValueError("gelu_tanh needs an even number of elements")
    out = torch.empty_like(xh)
    if n:
        with torch.cuda.device(xh.device):
            _lib.check(lib.vdmq_gelu_tanh_f16(xh.data_ptr(), out.data_ptr(), n, _k._stream(xh.device)))
    return out


def linear_gelu_vdm_w4a4(
    x: torch.Tensor,
    qweight: torch.Tensor,
    wscales: torch.Tensor,
    bias: Optional[torch.Tensor] = None,
    clip_ratio: float = 1.0,
    bias_half: Optional[torch.Tensor] = None,
) -> torch.Tensor:
    """``linear_vdm_w4a4(gelu_tanh(x), qweight, wscales, bias, clip_ratio, bias_half)``
    in two kernels instead of three; same argument conventions and errors as
    ``linear_vdm_w4a4`` (vdm_w4a4.py:222-244 of the reference)."""
    _k._load_ext()
    x_2d, orig_shape = _k._as_2d_half_contiguous(x)
    _k._check_linear_shapes(x_2d, qweight, wscales)
    _k._require(x_2d.is_cuda, "input must be a CUDA tensor")
    native_w, wscale = _k._native_weights(qweight.contiguous(), wscales.contiguous())
    b = bias_half if bias_half is not None else bias
    if b is not None:
        b = b.half().contiguous().view(-1)
    out = _k._linear_2d(x_2d, native_w, wscale, b, clip_ratio, act="gelu_tanh")
    return out.view(*orig_shape, -1)
