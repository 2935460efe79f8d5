"""``QuantLinear`` / ``UniformQuantizer`` with the reference's module API
(vdm_infer/quantization/quant_linear.py), so that a Wan transformer whose
``nn.Linear`` layers were swapped for ``QuantLinear`` runs unchanged.

Two forward modes, as in the reference:

* fake-quant mode (``use_vdm_kernel`` False): ``F.linear(aq(x), wq(w), bias)``
  with uniform quantize-dequantize in torch (quant_linear.py:173-178);
* kernel mode (``use_vdm_kernel`` True): the packed W4A4 path through
  ``dsaquant_amd.kernels.vdm_w4a4.linear_vdm_w4a4`` (quant_linear.py:163-172).

State-dict keys, buffer names and attribute names are the reference's.
"""
from __future__ import annotations

import torch
import torch.nn as nn
import torch.nn.functional as F

_GRANULARITY_VIEWS = {
    "per_tensor": lambda q, x: x.reshape(1, -1),
    "per_channel": lambda q, x: x.reshape(x.shape[0], -1),
    "per_token": lambda q, x: x.reshape(-1, x.shape[-1]),
    "per_group": lambda q, x: x.reshape(-1, q.group_size),
}


class UniformQuantizer(nn.Module):
    """Uniform (a)symmetric fake-quantizer; qparams are taken from the first
    tensor seen and then frozen (quant_linear.py:6-86)."""

    def __init__(self, bit: int = 4, sym: bool = True, granularity: str = "per_channel", group_size: int = -1,
                 round_zero: bool = True, cali: str = "mse", clip_ratio: float = 1.0, **kwargs) -> None:
        super().__init__()
        self.bit, self.sym = bit, sym
        self.granularity, self.group_size = granularity, group_size
        self.round_zero, self.cali, self.clip_ratio = round_zero, cali, clip_ratio
        # integer grid [N, P]
        self.P = (1 << (bit - 1)) - 1 if sym else (1 << bit) - 1
        self.N = -(1 << (bit - 1)) if sym else 0
        self.scale = None
        self.zero_point = None
        self.init = False

    def reshape(self, x: torch.Tensor) -> torch.Tensor:
        try:
            view = _GRANULARITY_VIEWS[self.granularity]
        except KeyError:
            raise ValueError(f"Unsupported granularity: {self.granularity}") from None
        return view(self, x)

    def _set_buffer(self, name: str, value) -> None:
        if hasattr(self, name):
            delattr(self, name)
        if value is None:
            setattr(self, name, None)
        else:
            self.register_buffer(name, value)

    def init_qparams(self, x: torch.Tensor) -> None:
        rows = self.reshape(x.float())
        lo = rows.amin(dim=-1, keepdim=True) * self.clip_ratio
        hi = rows.amax(dim=-1, keepdim=True) * self.clip_ratio
        if self.sym:
            scale = torch.maximum(lo.abs(), hi.abs()).clamp(min=1e-5) / self.P
            zero_point = None
        else:
            scale = ((hi - lo) / self.P).clamp_min(1e-9)
            zero_point = (-torch.round(lo / scale)).clamp(self.N, self.P)
        self._set_buffer("scale", scale.to(dtype=x.dtype))
        self._set_buffer("zero_point", None if zero_point is None else zero_point.to(dtype=x.dtype))
        self.init = True

    def quant(self, x: torch.Tensor, scale: torch.Tensor, zero_point):
        if zero_point is None:
            q = torch.round(x / scale)
        elif self.round_zero:
            q = torch.round(x / scale) + zero_point
        else:
            q = torch.round(x / scale + zero_point)
        return torch.clamp(q, self.N, self.P)

    def dequant(self, x: torch.Tensor, scale: torch.Tensor, zero_point):
        return x * scale if zero_point is None else scale * (x - zero_point)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        if not self.init or self.scale is None:
            self.init_qparams(x)
        rows = self.reshape(x)
        fake = self.dequant(self.quant(rows, self.scale, self.zero_point), self.scale, self.zero_point)
        return fake.reshape(x.shape)

    def build(self) -> None:
        if self.scale is not None:
            self.init = True


QuantizerMap = {name: UniformQuantizer for name in ("uniform", "lsq", "lsq+", "dynamic", "learnable_clipped_dynamic")}


class QuantLinear(nn.Module):
    """Drop-in for ``nn.Linear`` (quant_linear.py:98-181 of the reference)."""

    def __init__(self, layer: nn.Linear, quantizer_type: dict = {"w": "uniform", "act": "uniform"},
                 q_params: dict = {"w": {}, "act": {}}) -> None:
        super().__init__()
        self.kwd_func = F.linear
        self.weight = nn.Parameter(layer.weight.detach().clone())
        self.out_features, self.in_features = self.weight.shape
        self.bias = None if layer.bias is None else nn.Parameter(layer.bias.detach().clone())
        self.use_wq = False
        self.use_aq = False
        self.wquantizer = QuantizerMap[quantizer_type["w"]](**q_params["w"])
        self.aquantizer = QuantizerMap[quantizer_type["act"]](**q_params["act"])
        self.extra_repr_prefix = layer.extra_repr()
        self.use_hadamard = False
        self.use_timestep_scaling = False
        self.use_kernel = False
        self.use_kernel_fused = False
        self.use_vdm_kernel = False
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
        from dsaquant_amd.kernels.vdm_w4a4 import pack_weight_with_scale

        assert self.wquantizer is not None and self.wquantizer.scale is not None, "Weight quantizer scale is missing"
        assert self.wquantizer.sym, "Only symmetric quantization supported for VDM kernel"
        qweight, packed_scales, channel_scales = pack_weight_with_scale(self.weight.detach(), self.wquantizer.scale.detach().view(-1))
        self.register_buffer("vdm_weight_packed", qweight)
        self.register_buffer("vdm_weight_scale_packed", packed_scales)
        self.register_buffer("vdm_weight_scale", channel_scales.half())

    def enable_vdm_kernel_mode(self):
        """Switch to the packed kernel path and drop the fp weight
        (quant_linear.py:146-160).  Fails loudly if the HIP library is absent."""
        from dsaquant_amd.kernels.vdm_w4a4 import is_available, load_error

        assert is_available(), f"DSAQuant W4A4 kernel not compiled/available: {load_error()}"
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
            from dsaquant_amd.kernels.vdm_w4a4 import linear_vdm_w4a4

            return linear_vdm_w4a4(x, self.vdm_weight_packed, self.vdm_weight_scale_packed, self.bias, self.kernel_clip_ratio,
                                   bias_half=self._bias_half)
        w = self.weight
        if self.use_wq and self.wquantizer is not None:
            w = self.wquantizer(w)
        if self.use_aq and self.aquantizer is not None:
            x = self.aquantizer(x)
        return self.kwd_func(x, w, self.bias)

    def extra_repr(self) -> str:
        return f"{self.extra_repr_prefix}, use_aq={self.use_aq}, use_wq={self.use_wq}, use_vdm_kernel={self.use_vdm_kernel}"
