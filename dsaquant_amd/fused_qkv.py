"""Fused QKV / KV projection dispatch for attention modules, with the contract
of ``_get_qkv_projections`` in the reference's
vdm_infer/models/wan_vdm/modules/attention.py:35-121.

``attn`` is any module exposing ``to_q``, ``to_k``, ``to_v`` (QuantLinear in
kernel mode for the fused path), ``cross_attention_dim_head`` (None for
self-attention), ``use_fused_qkv_kernel`` and ``qkv_kernel_backend``; optional
``fused_projections`` / ``to_qkv`` / ``to_kv`` for the fp fused variant.

Self-attention: ONE activation quantization and ONE GEMM against the cached
row-concatenation Wq|Wk|Wv, split three ways.  Cross-attention: ``to_q`` on the
tokens, one fused K|V GEMM on the encoder states.  The concatenated weight is
relaid once from the projections' own packed buffers into the form the kernels
stream (no concatenated v1 copy is made); the concatenated bias is cached on
the module under the reference's attribute name (``_vdm_qkv_bias_half`` ...).
"""
from __future__ import annotations

from typing import List, Optional

import torch


def fused_parts(module):
    """Names of the projections whose packed weights ``module`` uses as ONE concatenated weight: q|k|v of a
    self-attention module and k|v of a cross-attention module once they are marked for the fused kernel path
    (packed_checkpoint.py:167-188 of the reference sets the marks); nothing for any other module."""
    if not (getattr(module, "use_fused_qkv_kernel", False) and getattr(module, "qkv_kernel_backend", None) == "vdm"):
        return []
    if not all(hasattr(module, n) and getattr(getattr(module, n), "vdm_weight_packed", None) is not None for n in ("to_q", "to_k", "to_v")):
        return []
    return [["to_q", "to_k", "to_v"]] if module.cross_attention_dim_head is None else [["to_k", "to_v"]]


def _cat_prepared(attn, names: List[str], prefix: str):
    """The concatenated weight of ``attn.<name>`` for the kernels and the concatenated fp16 bias (or None).  The
    reference caches concatenated v1 buffers on the module (``_vdm_qkv_weight_packed`` ..., attention.py:44-54); the
    kernels here never read a concatenated v1 buffer -- the operand is relaid from the projections' own buffers and
    kept with them -- so only the bias keeps its cache attribute."""
    from dsaquant_amd.kernels import vdm_w4a4 as k

    b_attr = f"_vdm_{prefix}_bias_half"
    layers = [getattr(attn, n) for n in names]
    weight = k._prepared([(l.vdm_weight_packed, l.vdm_weight_scale_packed) for l in layers])
    if getattr(attn, b_attr, None) is None:
        biases = [l._bias_half for l in layers]
        if any(b is not None for b in biases):
            n, dev = layers[0].vdm_weight_packed.shape[0], layers[0].vdm_weight_packed.device
            filled = [b if b is not None else torch.zeros(n, dtype=torch.float16, device=dev) for b in biases]
            setattr(attn, b_attr, torch.cat(filled, dim=0).contiguous())
        else:
            setattr(attn, b_attr, None)
    return weight, getattr(attn, b_attr)


def _project_cat(attn, names: List[str], prefix: str, x: torch.Tensor, clip_ratio: float):
    from dsaquant_amd.kernels import vdm_w4a4 as k

    weight, bias = _cat_prepared(attn, names, prefix)
    n = getattr(attn, names[0]).vdm_weight_packed.shape[0]
    if getattr(attn, "qkv_contiguous_outputs", True):
        # each projection's output as its own contiguous tensor, written in place by the GEMM epilogue: the values of
        # the reference's strided views (vdm_w4a4.py:297-298) without the strides
        return k.linear_vdm_w4a4_prepared(x, weight, bias, clip_ratio, split_cols=n).unbind(0)
    return k.linear_vdm_w4a4_prepared(x, weight, bias, clip_ratio).split(n, dim=-1)


def get_qkv_projections(attn, hidden_states: torch.Tensor, encoder_hidden_states: Optional[torch.Tensor]):
    if encoder_hidden_states is None:
        encoder_hidden_states = hidden_states

    if getattr(attn, "use_fused_qkv_kernel", False) and getattr(attn, "qkv_kernel_backend", None) == "vdm":
        if attn.cross_attention_dim_head is None:
            return tuple(_project_cat(attn, ["to_q", "to_k", "to_v"], "qkv", hidden_states, attn.to_q.kernel_clip_ratio))
        query = attn.to_q(hidden_states)
        key, value = _project_cat(attn, ["to_k", "to_v"], "kv", encoder_hidden_states, attn.to_k.kernel_clip_ratio)
        return query, key, value

    if getattr(attn, "fused_projections", False):
        if attn.cross_attention_dim_head is None:
            query, key, value = attn.to_qkv(hidden_states).chunk(3, dim=-1)
        else:
            query = attn.to_q(hidden_states)
            key, value = attn.to_kv(encoder_hidden_states).chunk(2, dim=-1)
        return query, key, value
    return attn.to_q(hidden_states), attn.to_k(encoder_hidden_states), attn.to_v(encoder_hidden_states)


# the reference's private name, for callers that import it as such
_get_qkv_projections = get_qkv_projections
