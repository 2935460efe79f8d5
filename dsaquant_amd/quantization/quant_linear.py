"""``QuantLinear`` / ``UniformQuantizer`` with the reference's module API
(vdm_infer/quantization/quant_linear.py), so that a Wan transformer whose
``nn.Linear`` layers were swapped for ``QuantLinear`` runs unchanged.

Two forward modes, as in the reference:

* fake-quant mode (``use_vdm_kernel`` False): ``F.linear(aq(x), wq(w), bias)``
  with uniform quantize-dequantize in torch (quant_linear.py:173-178);
* kernel mode (``use_vdm_kernel`` True): the packed W4A4 path through
  ``dsaquant_amd.kernels.vdm_w4a4.linear_vdm_w4a4`` (quant_linear.py:163-172).

State-dict keys, buffer names and attribute names are the reference's; the
arithmetic of the fake-quant mode is held to vectors recorded from the
reference (tests/golden/quantlinear_fp_path.npz).
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch
import torch.nn as nn
import torch.nn.functional as F


# ---------------------------------------------------------------- the quantizer's arithmetic, as plain functions

def _integer_grid(bit: int, sym: bool) -> Tuple[int, int]:
    """(lowest, highest) code: two's-complement range when symmetric, unsigned otherwise."""
    if sym:
        half = 1 << (bit - 1)
        return -half, half - 1
    return 0, (1 << bit) - 1


def _rows_view(x: torch.Tensor, granularity: str, group_size: int) -> torch.Tensor:
    """The 2-D view whose rows share one set of parameters (quant_linear.py:33-42).  Note "per_channel" keeps the
    FIRST axis: for a 2-D activation that is one row per token, for a 3-D one it is one row per batch element."""
    if granularity == "per_tensor":
        return x.reshape(1, -1)
    if granularity == "per_channel":
        return x.reshape(x.shape[0], -1)
    if granularity == "per_token":
        return x.reshape(-1, x.shape[-1])
    if granularity == "per_group":
        return x.reshape(-1, group_size)
    raise ValueError(f"Unsupported granularity: {granularity}")


def _row_parameters(rows_f32: torch.Tensor, clip: float, lowest: int, highest: int, sym: bool):
    """(scale, zero_point or None) in fp32 from the clipped row extrema (quant_linear.py:43-52)."""
    top = rows_f32.amax(dim=-1, keepdim=True) * clip
    bottom = rows_f32.amin(dim=-1, keepdim=True) * clip
    if sym:
        return torch.maximum(bottom.abs(), top.abs()).clamp(min=1e-5) / highest, None
    step = ((top - bottom) / highest).clamp_min(1e-9)
    return step, (-torch.round(bottom / step)).clamp(lowest, highest)


class UniformQuantizer(nn.Module):
    """Uniform (a)symmetric fake-quantizer; the parameters are taken from the first
    tensor seen and then frozen (quant_linear.py:6-86)."""

    def __init__(self, bit: int = 4, sym: bool = True, granularity: str = "per_channel", group_size: int = -1,
                 round_zero: bool = True, cali: str = "mse", clip_ratio: float = 1.0, **kwargs) -> None:
        super().__init__()
        self.N, self.P = _integer_grid(bit, sym)
        self.bit, self.sym, self.granularity, self.group_size = bit, sym, granularity, group_size
        self.round_zero, self.cali, self.clip_ratio = round_zero, cali, clip_ratio
        self.scale: Optional[torch.Tensor] = None
        self.zero_point: Optional[torch.Tensor] = None
        self.init = False

    def reshape(self, x: torch.Tensor) -> torch.Tensor:
        return _rows_view(x, self.granularity, self.group_size)

    def _replace(self, name: str, value: Optional[torch.Tensor]) -> None:
        # a plain None attribute and a registered buffer of the same name cannot coexist
        if hasattr(self, name):
            delattr(self, name)
        if value is None:
            setattr(self, name, None)
        else:
            self.register_buffer(name, value)

    def init_qparams(self, x: torch.Tensor) -> None:
        scale, zero_point = _row_parameters(self.reshape(x.float()), self.clip_ratio, self.N, self.P, self.sym)
        self._replace("scale", scale.to(dtype=x.dtype))
        self._replace("zero_point", None if zero_point is None else zero_point.to(dtype=x.dtype))
        self.init = True

    def quant(self, x: torch.Tensor, scale: torch.Tensor, zero_point):
        ratio = x / scale
        if zero_point is None:
            codes = torch.round(ratio)
        elif self.round_zero:
            codes = torch.round(ratio) + zero_point
        else:
            codes = torch.round(ratio + zero_point)
        return torch.clamp(codes, self.N, self.P)

    def dequant(self, x: torch.Tensor, scale: torch.Tensor, zero_point):
        return x * scale if zero_point is None else scale * (x - zero_point)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        if self.scale is None or not self.init:
            self.init_qparams(x)
        codes = self.quant(self.reshape(x), self.scale, self.zero_point)
        return self.dequant(codes, self.scale, self.zero_point).reshape(x.shape)

    def build(self) -> None:
        if self.scale is not None:
            self.init = True


QuantizerMap = dict.fromkeys(("uniform", "lsq", "lsq+", "dynamic", "learnable_clipped_dynamic"), UniformQuantizer)

# switches a fresh QuantLinear starts with, all off (quant_linear.py:111-120)
_SWITCHES = ("use_wq", "use_aq", "use_hadamard", "use_timestep_scaling", "use_kernel", "use_kernel_fused", "use_vdm_kernel")


def _kernels():
    from dsaquant_amd.kernels import vdm_w4a4

    return vdm_w4a4


class QuantLinear(nn.Module):
    """Drop-in for ``nn.Linear`` (quant_linear.py:98-181 of the reference)."""

    def __init__(self, layer: nn.Linear, quantizer_type: dict = {"w": "uniform", "act": "uniform"},
                 q_params: dict = {"w": {}, "act": {}}) -> None:
        super().__init__()
        self.kwd_func = F.linear
        self.extra_repr_prefix = layer.extra_repr()
        self.weight = nn.Parameter(layer.weight.detach().clone())
        self.bias = None if layer.bias is None else nn.Parameter(layer.bias.detach().clone())
        self.out_features, self.in_features = self.weight.shape
        for role, attr in (("w", "wquantizer"), ("act", "aquantizer")):
            setattr(self, attr, QuantizerMap[quantizer_type[role]](**q_params[role]))
        for switch in _SWITCHES:
            setattr(self, switch, False)
        self.kernel_clip_ratio = 0.95
        self._bias_half = None

    # -- switches ---------------------------------------------------------
    def set_quant_state(self, use_wq: bool = False, use_aq: bool = False) -> None:
        self.use_wq, self.use_aq = use_wq, use_aq

    def set_cur_timestep(self, t) -> None:
        self.cur_timestep = t

    def set_hadamard(self, use_hadamard: bool = False) -> None:
        if use_hadamard:
            raise NotImplementedError("Hadamard rotation is not included in the inference-only release.")
        self.use_hadamard = False

    # -- kernel mode ------------------------------------------------------
    def prepare_vdm_kernel_weights(self):
        """Quantize ``weight`` with the weight quantizer's per-channel scale and
        register the three packed buffers (quant_linear.py:136-144)."""
        wq = self.wquantizer
        assert wq is not None and wq.scale is not None, "Weight quantizer scale is missing"
        assert wq.sym, "Only symmetric quantization supported for VDM kernel"
        packed, packed_scales, channel_scales = _kernels().pack_weight_with_scale(self.weight.detach(), wq.scale.detach().view(-1))
        for name, tensor in (("vdm_weight_packed", packed), ("vdm_weight_scale_packed", packed_scales),
                             ("vdm_weight_scale", channel_scales.half())):
            self.register_buffer(name, tensor)

    def enable_vdm_kernel_mode(self):
        """Switch to the packed kernel path and drop the fp weight
        (quant_linear.py:146-160).  Fails loudly if the HIP library is absent."""
        k = _kernels()
        assert k.is_available(), f"DSAQuant W4A4 kernel not compiled/available: {k.load_error()}"
        if not hasattr(self, "vdm_weight_packed"):
            self.prepare_vdm_kernel_weights()
        self.use_vdm_kernel, self.use_kernel, self.use_kernel_fused = True, False, False
        if self.bias is not None:
            self._bias_half = self.bias.half().contiguous()
        if getattr(self, "weight", None) is not None:
            self.register_parameter("weight", None)
        if getattr(self, "wquantizer", None) is not None:
            del self.wquantizer
            self.wquantizer = None

    # -- forward ----------------------------------------------------------
    def forward(self, x: torch.Tensor) -> torch.Tensor:
        if self.use_vdm_kernel:
            return _kernels().linear_vdm_w4a4(x, self.vdm_weight_packed, self.vdm_weight_scale_packed, self.bias,
                                              self.kernel_clip_ratio, bias_half=self._bias_half)
        weight = self.wquantizer(self.weight) if self.use_wq and self.wquantizer is not None else self.weight
        if self.use_aq and self.aquantizer is not None:
            x = self.aquantizer(x)
        return self.kwd_func(x, weight, self.bias)

    def extra_repr(self) -> str:
        return f"{self.extra_repr_prefix}, use_aq={self.use_aq}, use_wq={self.use_wq}, use_vdm_kernel={self.use_vdm_kernel}"
