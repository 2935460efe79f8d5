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

``LnInput`` + ``linear_ln_vdm_w4a4`` / ``qkv_projections_ln`` do the same for
the block's ``norm(x) * (1 + scale) + shift`` (dit_block.py:100, :110) and for
the affine ``norm2`` (:105): the LayerNorm, the modulation and the quantizer
become one pass over ``x``.  ``linear_fused`` adds the consumer side: the gated
residual update ``hidden_states + y * gate`` (:102, :107, :112) in the GEMM epilogue.
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
    return linear_fused(x, qweight, wscales, bias, clip_ratio, bias_half, act="gelu_tanh")


class LnInput:
    """A linear's input that is still to be produced: ``LayerNorm(x)`` followed by
    the modulation ``* (1 + a) + b`` (``mode="modulate"``, a = scale, b = shift,
    fp16 arithmetic on the fp16 LayerNorm output) or by the affine ``* a + b``
    (``mode="affine"``, a = weight, b = bias, fp32 arithmetic, one rounding).

    ``x`` is ``[B, L, K]`` (or ``[L, K]``); ``a`` and ``b`` hold one vector per batch
    element (``[B, K]``, ``[B, 1, K]`` or ``[K]``) or one per token (``[B, L, K]``).
    """

    def __init__(self, x: torch.Tensor, a: torch.Tensor, b: torch.Tensor, eps: float, mode: str = "modulate"):
        if mode not in ("modulate", "affine"):
            raise ValueError(f"unknown LayerNorm mode {mode!r}")
        self.shape = tuple(x.shape)
        K = x.shape[-1]
        self.x = x.reshape(-1, K).half().contiguous()
        M = self.x.shape[0]
        a2, b2 = a.reshape(-1, K).half().contiguous(), b.reshape(-1, K).half().contiguous()
        if a2.shape != b2.shape:
            raise ValueError("the two LayerNorm vectors must have the same shape")
        nvec = a2.shape[0]
        if nvec == 0 or M % nvec != 0:
            raise ValueError(f"{nvec} vectors do not divide {M} rows")
        self.a, self.b, self.rows_per_vec = a2, b2, M // nvec
        self.eps, self.mode = float(eps), mode
        self.code = _lib.VDMQ_LN_MODULATE if mode == "modulate" else _lib.VDMQ_LN_AFFINE

    def _args(self):
        M, K = self.x.shape
        return (self.x.data_ptr(), M, K, self.x.stride(0), self.eps, self.code, self.a.data_ptr(), self.b.data_ptr(), self.a.stride(0),
                self.rows_per_vec)

    def materialize(self) -> torch.Tensor:
        """The fp16 tensor the fused quantizer sees (same kernel arithmetic), shaped like ``x``."""
        lib = _k._load_ext()
        _k._check_device_tensor(self.x, "input", torch.float16)
        h = torch.empty_like(self.x)
        if h.numel():
            with torch.cuda.device(h.device):
                _lib.check(lib.vdmq_ln_f16(*self._args(), h.data_ptr(), h.stride(0), _k._stream(h.device)))
        return h.view(self.shape)

    def quantize(self, clip_ratio: float = 1.0, bf6: bool = False):
        """``(qact native, scales)`` of the produced input, as ``quantize_activation_native`` returns them
        (``bf6=True``: as ``quantize_activation_bf6`` does)."""
        lib = _k._load_ext()
        _k._check_device_tensor(self.x, "input", torch.float16)
        M, K = self.x.shape
        dev = self.x.device
        if bf6:
            with torch.cuda.device(dev):
                return _k._quantize_for_gemm(self.x, clip_ratio, 0, True, self._args())
        with torch.cuda.device(dev):
            native = torch.empty((M, _k.k_padded(K) // 2), dtype=torch.uint8, device=dev)
            scales = torch.empty((M,), dtype=torch.float16, device=dev)
            if M:
                _lib.check(lib.vdmq_quantize_act_ln(*self._args(), float(clip_ratio), native.data_ptr(), scales.data_ptr(), _k._stream(dev)))
        return native, scales


def linear_ln_vdm_w4a4(
    pre: LnInput,
    qweight: torch.Tensor,
    wscales: torch.Tensor,
    bias: Optional[torch.Tensor] = None,
    clip_ratio: float = 1.0,
    bias_half: Optional[torch.Tensor] = None,
) -> torch.Tensor:
    """``linear_vdm_w4a4(pre.materialize(), ...)`` without materializing: LayerNorm,
    modulation and activation quantizer are one kernel, the GEMM the second."""
    return linear_fused(pre, qweight, wscales, bias, clip_ratio, bias_half)


class QuantizedInput:
    """A linear's input that is already quantized per token (fp16 scales and the operand form
    of the matrix path its row length takes: 6-bit blocks or native int4 rows): one quantizer
    launch serves every linear that reads the same tensor with the same clip ratio.  The
    cross-attention context is such a tensor -- every block's ``attn2`` K/V projection reads
    ``encoder_hidden_states`` (dit_block.py:109 of the reference), which the reference
    quantizes again in each of them."""

    def __init__(self, x: torch.Tensor, clip_ratio: float = 1.0):
        self.shape = tuple(x.shape)
        self.clip_ratio = float(clip_ratio)
        x_2d, _ = _k._as_2d_half_contiguous(x)
        _k._require(x_2d.is_cuda, "input must be a CUDA tensor")
        self.M, self.K = x_2d.shape
        self.device = x_2d.device
        # (the path of a linear depends on its row length alone, so it is known before any weight is)
        self.bf6 = _k._use_bf6(self.M, 128, self.K)
        if self.M:
            self.qact, self.scales = _k._quantize_for_gemm(x_2d, self.clip_ratio, _lib.VDMQ_ACT_NONE, self.bf6, None)
        else:
            self.qact = self.scales = None


def linear_fused(
    x,
    qweight,
    wscales: Optional[torch.Tensor],
    bias: Optional[torch.Tensor] = None,
    clip_ratio: float = 1.0,
    bias_half: Optional[torch.Tensor] = None,
    *,
    act: Optional[str] = None,
    residual: Optional[torch.Tensor] = None,
    gate: Optional[torch.Tensor] = None,
    split_cols: Optional[int] = None,
) -> torch.Tensor:
    """``residual + linear_vdm_w4a4(act(x), ...) * gate`` in two kernels.

    ``x`` is a tensor (optionally with ``act="gelu_tanh"`` applied to it inside the
    quantizer), an ``LnInput`` or a ``QuantizedInput`` (whose clip ratio must be the
    layer's; the GEMM then runs on the matrix path the input was quantized for).  ``gate`` (fp16, one ``[N]`` vector per batch element
    or per token) and ``residual`` (fp16, shaped like the output) are folded into the
    GEMM epilogue as the two fp16 tensor operations of the reference's
    ``hidden_states + attn_output * gate`` (dit_block.py:102, :107, :112); either may
    be omitted.  ``qweight`` may be a ``PreparedWeight`` (then ``wscales`` is ignored): the concatenated weight of a
    fused projection.  ``split_cols``: the output columns as N / split_cols contiguous tensors, stacked in front
    (``[N / split_cols, ..., split_cols]``; without gate and residual).  Returns a new tensor; nothing is updated in place."""
    _k._load_ext()  # raises when the library is missing
    if isinstance(x, LnInput):
        if act is not None:
            raise ValueError("an activation cannot be combined with a LayerNorm input")
        pre, x_2d, lead = x, x.x, x.shape[:-1]
    elif isinstance(x, QuantizedInput):
        if act is not None:
            raise ValueError("an activation cannot be applied to an input that is already quantized")
        if x.clip_ratio != float(clip_ratio):
            raise ValueError(f"input quantized with clip ratio {x.clip_ratio}, the layer wants {float(clip_ratio)}")
        pre, x_2d, lead = x, None, x.shape[:-1]
    else:
        pre = None
        x_2d, lead = _k._as_2d_half_contiguous(x)
    prepared = isinstance(qweight, _k.PreparedWeight)
    if x_2d is not None:
        _k._require(x_2d.is_cuda, "input must be a CUDA tensor")
        M, K = x_2d.shape
        dev = x_2d.device
    else:
        M, K, dev = pre.M, pre.K, pre.device
    if prepared:
        if qweight.K != K:
            raise ValueError("qweight shape must be [N, K/2]")
    else:
        _k._check_packed_weight(qweight, wscales, K)
    act_code = _k._act_code(act)
    weight = qweight if prepared else _k._prepared_weight(qweight, wscales)
    N = weight.N
    b = bias_half if bias_half is not None else bias
    if b is not None:
        b = b.half().contiguous().view(-1)
        _k._check_device_tensor(b, "bias", torch.float16)
        _k._require(b.numel() == N, "bias length must equal N")
    g2 = r2 = None
    rows_per_gate = 1
    if gate is not None:
        if gate.shape[-1] != N:
            raise ValueError(f"gate must have {N} channels")
        g2 = gate.reshape(-1, N).half().contiguous()
        _k._check_device_tensor(g2, "gate", torch.float16)
        if g2.shape[0] == 0 or (M and M % g2.shape[0] != 0):
            raise ValueError(f"{g2.shape[0]} gate vectors do not divide {M} rows")
        rows_per_gate = max(1, M // g2.shape[0])
    if residual is not None:
        if tuple(residual.shape) != tuple(lead) + (N,):
            raise ValueError(f"residual must have shape {tuple(lead) + (N,)}, got {tuple(residual.shape)}")
        r2 = residual.reshape(-1, N).half().contiguous()
        _k._check_device_tensor(r2, "residual", torch.float16)
    if split_cols is not None:
        if gate is not None or residual is not None:
            raise ValueError("a split output takes neither gate nor residual")
        if split_cols <= 0 or split_cols % 64 != 0 or N % split_cols != 0:
            raise ValueError(f"split_cols must be a positive multiple of 64 that divides N={N} (got {split_cols})")
    with torch.cuda.device(dev):
        out = torch.empty((M, N) if split_cols is None else (N // split_cols, M, split_cols), dtype=torch.float16, device=dev)
        if M and isinstance(pre, QuantizedInput):
            _k._gemm_dispatch(pre.qact, pre.scales, pre.bf6, weight, b, out, K, gate=g2, rows_per_gate=rows_per_gate, residual=r2)
        elif M:
            bf6 = _k._use_bf6(M, N, K)
            operand, scales = _k._quantize_for_gemm(x_2d, clip_ratio, act_code, bf6, None if pre is None else pre._args())
            _k._gemm_dispatch(operand, scales, bf6, weight, b, out, K, gate=g2, rows_per_gate=rows_per_gate, residual=r2)
    return out.view(*lead, N) if split_cols is None else out.view(N // split_cols, *lead, split_cols)


def qkv_projections_ln(attn, pre: LnInput):
    """Self-attention Q, K, V of ``pre`` through the cached concatenation Wq|Wk|Wv
    (the fused branch of ``get_qkv_projections``, attention.py:41-68 of the
    reference) with the LayerNorm fused into the one activation quantization."""
    from .fused_qkv import _cat_prepared

    w, b = _cat_prepared(attn, ["to_q", "to_k", "to_v"], "qkv")
    n = attn.to_q.vdm_weight_packed.shape[0]
    if getattr(attn, "qkv_contiguous_outputs", False):
        return linear_fused(pre, w, None, None, attn.to_q.kernel_clip_ratio, bias_half=b, split_cols=n).unbind(0)
    return linear_ln_vdm_w4a4(pre, w, None, None, attn.to_q.kernel_clip_ratio, bias_half=b).split(n, dim=-1)


def kv_projections(attn, encoder_hidden_states):
    """Cross-attention K, V through the cached concatenation Wk|Wv (attention.py:70-107 of the reference);
    ``encoder_hidden_states`` is the tensor or a ``QuantizedInput`` of it shared between blocks."""
    from .fused_qkv import _cat_prepared

    w, b = _cat_prepared(attn, ["to_k", "to_v"], "kv")
    n = attn.to_k.vdm_weight_packed.shape[0]
    if getattr(attn, "qkv_contiguous_outputs", False):
        return linear_fused(encoder_hidden_states, w, None, None, attn.to_k.kernel_clip_ratio, bias_half=b, split_cols=n).unbind(0)
    return linear_fused(encoder_hidden_states, w, None, None, attn.to_k.kernel_clip_ratio, bias_half=b).split(n, dim=-1)
