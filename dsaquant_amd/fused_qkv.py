"""Fused QKV / KV projection dispatch for attention modules, with the contract
of ``_get_qkv_projections`` in the reference's
vdm_infer/models/wan_vdm/modules/attention.py:35-121.

``attn`` is any module exposing ``to_q``, ``to_k``, ``to_v`` (QuantLinear in
kernel mode for the fused path), ``cross_attention_dim_head`` (None for
self-attention), ``use_fused_qkv_kernel`` and ``qkv_kernel_backend``; optional
``fused_projections`` / ``to_qkv`` / ``to_kv`` for the fp fused variant.

Self-attention: ONE activation quantization and ONE GEMM against the cached
row-concatenation Wq|Wk|Wv, split three ways.  Cross-attention: ``to_q`` on the
tokens, one fused K|V GEMM on the encoder states.  The concatenated buffers are
built on first use and cached on the module under the reference's attribute
names (``_vdm_qkv_weight_packed`` ...).
"""
from __future__ import annotations

from typing import List, Optional

import torch


def _cat_cached(attn, names: List[str], prefix: str):
    """Concatenate the v1 buffers / biases of ``attn.<name>`` once and cache them."""
    w_attr, s_attr, b_attr = f"_vdm_{prefix}_weight_packed", f"_vdm_{prefix}_weight_scale", f"_vdm_{prefix}_bias_half"
    layers = [getattr(attn, n) for n in names]
    if getattr(attn, w_attr, None) is None:
        setattr(attn, w_attr, torch.cat([l.vdm_weight_packed for l in layers], dim=0).contiguous())
        setattr(attn, s_attr, torch.cat([l.vdm_weight_scale_packed for l in layers], dim=0).contiguous())
    if getattr(attn, b_attr, None) is None:
        biases = [l._bias_half for l in layers]
        if any(b is not None for b in biases):
            n, dev = layers[0].vdm_weight_packed.shape[0], layers[0].vdm_weight_packed.device
            filled = [b if b is not None else torch.zeros(n, dtype=torch.float16, device=dev) for b in biases]
            setattr(attn, b_attr, torch.cat(filled, dim=0).contiguous())
        else:
            setattr(attn, b_attr, None)
    return getattr(attn, w_attr), getattr(attn, s_attr), getattr(attn, b_attr)


def get_qkv_projections(attn, hidden_states: torch.Tensor, encoder_hidden_states: Optional[torch.Tensor]):
    if encoder_hidden_states is None:
        encoder_hidden_states = hidden_states

    if getattr(attn, "use_fused_qkv_kernel", False) and getattr(attn, "qkv_kernel_backend", None) == "vdm":
        from dsaquant_amd.kernels.vdm_w4a4 import linear_vdm_w4a4, linear_vdm_w4a4_qkv

        if attn.cross_attention_dim_head is None:
            w, s, b = _cat_cached(attn, ["to_q", "to_k", "to_v"], "qkv")
            q, k, v = attn.to_q, attn.to_k, attn.to_v
            return tuple(linear_vdm_w4a4_qkv(
                hidden_states,
                q.vdm_weight_packed, q.vdm_weight_scale_packed,
                k.vdm_weight_packed, k.vdm_weight_scale_packed,
                v.vdm_weight_packed, v.vdm_weight_scale_packed,
                clip_ratio=q.kernel_clip_ratio, w_qkv_packed=w, w_qkv_scale=s, qkv_bias_half=b))
        query = attn.to_q(hidden_states)
        w, s, b = _cat_cached(attn, ["to_k", "to_v"], "kv")
        kv = linear_vdm_w4a4(encoder_hidden_states, w, s, bias=None, clip_ratio=attn.to_k.kernel_clip_ratio, bias_half=b)
        key, value = kv.split(attn.to_k.vdm_weight_packed.shape[0], dim=-1)
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
