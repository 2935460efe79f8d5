"""``vdm_w4a4_packed_v1`` checkpoints: reader, writer and the switches that put
a model into kernel mode.  Same functions, arguments, return values and
exception types as the reference's vdm_infer/checkpoints/packed_checkpoint.py.

On disk a packed checkpoint is ``torch.save`` of
``{"format": "vdm_w4a4_packed_v1", "metadata": {...}, "model": state_dict}``
where, for every QuantLinear ``<name>``, the state dict holds
``<name>.vdm_weight_packed`` (u8 [N, K/2]), ``<name>.vdm_weight_scale_packed``
(fp16 [N, K/64]), ``<name>.vdm_weight_scale`` (fp16 [N]) and ``<name>.bias``
but no fp ``<name>.weight`` and no quantizer state.  Buffers stay in the v1
byte layout in the module (they are the state-dict contract); the loader
relays each of them once, as it puts the model on the GPU, into the one form
the gfx950 kernels stream for that layer (bf6 blocks or native int4 rows,
3/4 or 1/2 byte per weight beside the v1 buffer).
"""
from __future__ import annotations

import gc
from typing import Any

import torch
import torch.nn as nn

PACKED_CHECKPOINT_FORMAT = "vdm_w4a4_packed_v1"
# checkpoints written by earlier tooling carry another format string and other
# names for the three buffers (packed_checkpoint.py:19,25)
_LEGACY_PACKED_CHECKPOINT_FORMAT = "vdm_diy_w4a4_packed_v1"
VDM_BUFFER_SUFFIXES = ("vdm_weight_packed", "vdm_weight_scale_packed", "vdm_weight_scale")
_LEGACY_BUFFER_SUFFIXES = ("diy_weight_packed", "diy_weight_scale_packed", "diy_weight_scale")
_KNOWN_FORMATS = (PACKED_CHECKPOINT_FORMAT, _LEGACY_PACKED_CHECKPOINT_FORMAT)


def is_packed_checkpoint(ckpt: Any) -> bool:
    return isinstance(ckpt, dict) and "model" in ckpt and ckpt.get("format") in _KNOWN_FORMATS


def load_quant_checkpoint(path: str, dcp_loader) -> dict:
    """``.pt``/``.pth`` files are read with ``weights_only=True``; anything else
    is handed to ``dcp_loader`` (packed_checkpoint.py:32-37)."""
    if path.endswith((".pt", ".pth")):
        print(f"Loading torch checkpoint from {path}")
        return torch.load(path, map_location="cpu", weights_only=True)
    return dcp_loader(path)


def _key(module_name: str, suffix: str) -> str:
    return f"{module_name}.{suffix}" if module_name else suffix


def _is_quantizer_state(key: str) -> bool:
    return ".wquantizer." in key or ".aquantizer." in key


def _attach_buffer(module: nn.Module, name: str, tensor: torch.Tensor) -> None:
    module._buffers.pop(name, None)
    if hasattr(module, name):
        delattr(module, name)
    module.register_buffer(name, tensor.detach().contiguous())


def _to_kernel_mode(module: nn.Module) -> None:
    """Module state after packed buffers are attached (packed_checkpoint.py:120-131)."""
    module.use_vdm_kernel, module.use_kernel, module.use_kernel_fused = True, False, False
    module.set_quant_state(use_wq=True, use_aq=True)
    if getattr(module, "weight", None) is not None:
        module.register_parameter("weight", None)
    for q in ("wquantizer", "aquantizer"):
        if hasattr(module, q):
            delattr(module, q)
            setattr(module, q, None)


def _found_format(ckpt: Any):
    return ckpt.get("format") if isinstance(ckpt, dict) else type(ckpt)


def _stored_names(layer_name: str, state_dict: dict) -> dict:
    """buffer name -> the key it is stored under: the current name if present, else the legacy one."""
    names = {}
    for current, legacy in zip(VDM_BUFFER_SUFFIXES, _LEGACY_BUFFER_SUFFIXES):
        key = _key(layer_name, current)
        names[current] = key if key in state_dict else _key(layer_name, legacy)
    return names


def _ordinary_entries(state_dict: dict, fp_weight_keys: set) -> dict:
    """What goes through load_state_dict: everything but packed buffers (either naming), quantizer state, cached
    fp16 biases and the fp weights of the quantized layers (packed_checkpoint.py:84-93)."""
    packed = VDM_BUFFER_SUFFIXES + _LEGACY_BUFFER_SUFFIXES
    skip = lambda k: k.endswith(packed) or _is_quantizer_state(k) or k.endswith("._bias_half") or k in fp_weight_keys  # noqa: E731
    return {k: v for k, v in state_dict.items() if not skip(k)}


def load_packed_quantized_model(model: nn.Module, packed_ckpt: dict, *, quant_linear_cls: type, dtype: torch.dtype,
                                device: torch.device, require_vdm_kernel: bool = True, release_v1: bool = False) -> tuple:
    """Populate a freshly built model (Linear layers already swapped for
    ``quant_linear_cls``) from a packed checkpoint; returns ``(missing,
    unexpected)`` key lists (packed_checkpoint.py:52-148).

    Raises ValueError for an unknown format, AssertionError when the kernel
    library is required but unavailable, KeyError when a QuantLinear lacks any of
    its three buffers, RuntimeError when no QuantLinear was populated.  ``release_v1``
    (not in the reference): once every packed weight is relaid into the form the
    kernels stream, free the memory of the v1 weight buffers -- ``state_dict()``
    rebuilds them, see ``vdm_w4a4.release_v1_storage``.  The outcome
    on a file the reference's writer wrote is held to what the reference's loader
    leaves behind (tests/golden/reference_loader_outcome.json).
    """
    if not is_packed_checkpoint(packed_ckpt):
        raise ValueError(f"Unsupported checkpoint format: {_found_format(packed_ckpt)}")
    if require_vdm_kernel:
        from dsaquant_amd.kernels.vdm_w4a4 import is_available, load_error

        assert is_available(), f"DSAQuant W4A4 kernel not compiled/available: {load_error()}"

    state_dict = packed_ckpt["model"]
    quant_layers = {name: m for name, m in model.named_modules() if isinstance(m, quant_linear_cls)}
    fp_weight_keys = {_key(name, "weight") for name in quant_layers}

    # 1. everything that is not W4A4 state, through the ordinary route
    report = model.load_state_dict(_ordinary_entries(state_dict, fp_weight_keys), strict=False, assign=True)
    missing = [k for k in report.missing_keys if k not in fp_weight_keys and not _is_quantizer_state(k)]

    # 2. the packed buffers, attached layer by layer; a layer with any buffer absent is reported, not half-loaded
    absent: list = []
    populated = 0
    for name, module in quant_layers.items():
        stored = _stored_names(name, state_dict)
        gone = [key for key in stored.values() if key not in state_dict]
        if gone:
            absent += gone
            continue
        for buffer_name, key in stored.items():
            _attach_buffer(module, buffer_name, state_dict[key])
        _to_kernel_mode(module)
        populated += 1
    if absent:
        raise KeyError(f"Packed checkpoint is missing {len(absent)} VDM buffers, e.g. {', '.join(absent[:8])}")
    if not populated:
        raise RuntimeError("No QuantLinear layers were populated from the packed checkpoint")

    del state_dict
    gc.collect()

    # 3. dtype / device, then the fp16 bias each kernel call takes
    model = model.to(dtype).to(device)
    for module in model.modules():
        if isinstance(module, quant_linear_cls) and module.bias is not None:
            module._bias_half = module.bias.half().contiguous()
    _prepare_for_kernels(model, device, release_v1)
    print(f"Loaded packed DSAQuant W4A4 checkpoint: {populated} QuantLinear layers")
    return list(missing), list(report.unexpected_keys)


def _prepare_for_kernels(model: nn.Module, device, release_v1: bool = False) -> None:
    """The point at which the reference has its buffers attached and on the device (packed_checkpoint.py:102-148):
    relay them now, on the current stream, rather than inside the first forward (which may be under graph
    capture).  Nothing to do on a machine without the kernel library or for a model kept on the CPU."""
    if torch.device(device).type != "cuda":
        return
    from dsaquant_amd.kernels import vdm_w4a4

    if vdm_w4a4.is_available():
        vdm_w4a4.prepare_model(model)
        if release_v1:
            vdm_w4a4.release_v1_storage(model)


def enable_quant_kernels(model: nn.Module, *, quant_linear_cls: type) -> None:
    """Pack and switch every QuantLinear; a failing layer is reported and left
    in fake-quant mode (packed_checkpoint.py:151-164)."""
    print("Enabling DSAQuant W4A4 kernel mode...")
    for name, module in model.named_modules():
        if isinstance(module, quant_linear_cls):
            module.set_quant_state(use_wq=True, use_aq=True)
            try:
                module.enable_vdm_kernel_mode()
            except Exception as exc:
                print(f"  Failed to enable VDM kernel for {name}: {exc}")


def enable_fused_qkv(model: nn.Module, *, quant_linear_cls: type, attention_cls: type, use_fused_qkv: bool) -> None:
    """Mark attention modules whose q/k/v are all in kernel mode for the fused
    QKV path (packed_checkpoint.py:167-188)."""
    if not use_fused_qkv:
        return
    print("Enabling fused QKV kernel (vdm)...")
    for module in model.modules():
        if not isinstance(module, attention_cls):
            continue
        qkv = (module.to_q, module.to_k, module.to_v)
        if all(isinstance(p, quant_linear_cls) and p.use_vdm_kernel for p in qkv):
            module.use_fused_qkv_kernel = True
            module.qkv_kernel_backend = "vdm"
            _prepare_fused(module)


def _prepare_fused(attention: nn.Module) -> None:
    """The concatenated q|k|v (self-attention) or k|v (cross-attention) weight in the kernels' form, relaid from the
    projections' packed buffers; those projections are never called on their own from now on, so what was prepared
    for each of them alone is released."""
    from dsaquant_amd.fused_qkv import fused_parts
    from dsaquant_amd.kernels import vdm_w4a4

    for names in fused_parts(attention):
        layers = [getattr(attention, n) for n in names]
        if not all(l.vdm_weight_packed.is_cuda for l in layers) or not vdm_w4a4.is_available():
            continue
        lean = any("_vdmq_v1_released" in l.vdm_weight_packed.__dict__ for l in layers)
        vdm_w4a4.prepare_model(attention)  # (makes the concatenation; the projections' own forms go with their old buffers)
        if lean:
            vdm_w4a4.release_v1_storage(attention)


def packed_state_dict_from_model(model: nn.Module, *, float_dtype: torch.dtype = torch.float16) -> dict:
    """State dict for export: quantizer state and cached fp16 biases dropped,
    floating tensors cast to ``float_dtype``, uint8 kept (packed_checkpoint.py:190-199)."""
    out = {}
    for k, v in model.state_dict().items():
        if _is_quantizer_state(k) or k.endswith("._bias_half"):
            continue
        t = v.detach().cpu().contiguous()
        out[k] = t.to(float_dtype) if t.is_floating_point() else t
    return out


def save_packed_checkpoint(model: nn.Module, output_path: str, *, metadata: dict | None = None,
                           float_dtype: torch.dtype = torch.float16) -> None:
    torch.save({"format": PACKED_CHECKPOINT_FORMAT, "metadata": metadata or {},
                "model": packed_state_dict_from_model(model, float_dtype=float_dtype)}, output_path)
    print(f"Saved packed checkpoint to {output_path}")
