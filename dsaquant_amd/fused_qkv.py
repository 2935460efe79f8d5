"""Fused QKV / KV projection dispatch for attention modules, with the contract
of ``_get_qkv_projections`` in the reference's
vdm_infer/models/wan_vdm/modules/attention.py:35-121.

``attn`` is any module exposing ``to_q``, ``to_k``, ``to_v`` (QuantLinear in
kernel mode for the fused path), ``cross_attention_dim_head`` (None for
self-attention), ``use_fused_qkv_kernel`` and ``qkv_kernel_backend``; optional
``fused_projections`` / ``to_qkv`` / ``to_kv`` for the fp fused variant.

Self-attention: ONE activation quantization and ONE GEMM against the cached
row-concatenation Wq|Wk|Wv, split three ways.  Cross-attention: ``to_q`` on the
tokens, one fused K|V GEMM on the encoder states.  The concatenated v1 buffers
and the concatenated bias are cached on the module under the reference's
attribute names (``_vdm_qkv_weight_packed``, ``_vdm_qkv_weight_scale``,
``_vdm_qkv_bias_half``, ``_vdm_kv_*``), made at first need like there
(attention.py:44-66, 80-98); the projections' own buffers then become views of
the concatenation, so the weights are not held twice.  Results are three views
of one ``[..., 3N]`` tensor as in the reference; a module with
``qkv_contiguous_outputs = True`` gets three contiguous tensors instead (the
GEMM epilogue writes them in place: the same bits).
"""
from __future__ import annotations

import weakref
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


_PREFIX = {("to_q", "to_k", "to_v"): "qkv", ("to_k", "to_v"): "kv"}


def concatenated(attn, names: List[str]):
    """``(attn._vdm_<qkv|kv>_weight_packed, attn._vdm_<qkv|kv>_weight_scale)``: the row-concatenation of the
    projections' v1 weight and scale buffers, cached on the module under the names the reference uses and made when
    first needed (attention.py:44-54, 80-88).  Where the projections hold their buffers as registered buffers these
    are then replaced by views of the concatenation (same values, shapes and state-dict entries; one copy of the
    weights instead of two).  The cache is made anew when a projection's buffer is no longer such a view, e.g.
    after ``model.to(...)`` or a checkpoint load replaced it -- the projections' buffers are what counts."""
    from dsaquant_amd.kernels import vdm_w4a4 as k

    prefix = _PREFIX[tuple(names)]
    w_attr, s_attr = f"_vdm_{prefix}_weight_packed", f"_vdm_{prefix}_weight_scale"
    layers = [getattr(attn, n) for n in names]
    cat_w, cat_s = getattr(attn, w_attr, None), getattr(attn, s_attr, None)
    if cat_w is not None and cat_s is not None:
        owners = [l.vdm_weight_packed.__dict__.get("_vdmq_v1_owner") for l in layers]
        views = all(o is not None and o() is cat_w for o in owners)
        copies = all(o is None for o in owners) and getattr(attn, "_vdm_cat_is_copy", False) and cat_w.device == layers[0].vdm_weight_packed.device
        if views or copies:
            return cat_w, cat_s
    for l in layers:
        k.ensure_v1(l.vdm_weight_packed)
    cat_w = torch.cat([l.vdm_weight_packed for l in layers], dim=0).contiguous()
    cat_s = torch.cat([l.vdm_weight_scale_packed for l in layers], dim=0).contiguous()
    shared = all("vdm_weight_packed" in getattr(l, "_buffers", {}) for l in layers)
    row = 0
    for l in layers:
        n = l.vdm_weight_packed.shape[0]
        if shared:
            if l.vdm_weight_packed.is_cuda and k.is_available():
                k.release_prepared(l.vdm_weight_packed, concatenations=True)  # the old tensor's forms go with it
            view_w, view_s = cat_w[row:row + n], cat_s[row:row + n]
            view_w.__dict__["_vdmq_v1_owner"] = weakref.ref(cat_w)
            l._buffers["vdm_weight_packed"], l._buffers["vdm_weight_scale_packed"] = view_w, view_s
        row += n
    attn._vdm_cat_is_copy = not shared
    setattr(attn, w_attr, cat_w)
    setattr(attn, s_attr, cat_s)
    return cat_w, cat_s


def _cat_prepared(attn, names: List[str], prefix: str):
    """The concatenated weight of ``attn.<name>`` in the kernels' form and the concatenated fp16 bias (or None), the
    latter cached as ``_vdm_<prefix>_bias_half`` (attention.py:55-66, 89-98)."""
    from dsaquant_amd.kernels import vdm_w4a4 as k

    b_attr = f"_vdm_{prefix}_bias_half"
    layers = [getattr(attn, n) for n in names]
    weight = k._prepared_weight(*concatenated(attn, names))
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
    if getattr(attn, "qkv_contiguous_outputs", False):
        # opt-in: each projection's output as its own contiguous tensor, written in place by the GEMM epilogue -- the
        # values of the reference's strided views (vdm_w4a4.py:297-298) without the strides
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
