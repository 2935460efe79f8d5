#!/usr/bin/env python3
"""Writes tests/golden/reference_written_packed_v1.pt, reference_written_packed_legacy.pt and
reference_loader_outcome.json: a small `vdm_w4a4_packed_v1` checkpoint written by the reference's own
`save_packed_checkpoint`, and what the reference's own `load_packed_quantized_model` makes of it.

Nothing else pins the checkpoint reader / writer against the reference (its tests hold no checkpoint), so
this script loads two reference files by path on the CPU -- vdm_infer/quantization/quant_linear.py and
vdm_infer/checkpoints/packed_checkpoint.py -- builds the toy model below from the reference's QuantLinear,
gives its layers real packed buffers (the int4 weights under the weight quantizer's scale, laid out by the
oracle's v1 packers, as the reference's prepare_vdm_kernel_weights would through its CUDA packer), and
records the files and the outcome.  It runs only where the reference tree is present; the tests read the
committed files and never the reference.

    python tests/golden/make_checkpoint_fixture.py [/root/reference]
"""
import importlib.util
import json
import sys
from pathlib import Path

import torch
import torch.nn as nn

ROOT = Path(__file__).resolve().parents[2]
HERE = Path(__file__).resolve().parent
sys.path.insert(0, str(ROOT))
from tests.toy_model import build_toy  # noqa: E402  (the tests build the same model from this repository's QuantLinear)


def load_by_path(name: str, path: Path):
    # The reference tree is read-only by agreement: without this, the loader would leave a __pycache__ beside the file.
    sys.dont_write_bytecode = True
    spec = importlib.util.spec_from_file_location(name, path)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def describe(model: nn.Module, quant_linear_cls) -> dict:
    layers = {}
    for name, m in model.named_modules():
        if isinstance(m, quant_linear_cls):
            layers[name] = {
                "use_vdm_kernel": bool(m.use_vdm_kernel), "use_kernel": bool(m.use_kernel), "use_kernel_fused": bool(m.use_kernel_fused),
                "use_wq": bool(m.use_wq), "use_aq": bool(m.use_aq), "weight_is_none": m.weight is None,
                "wquantizer_is_none": m.wquantizer is None, "aquantizer_is_none": m.aquantizer is None,
                "bias_half": None if m._bias_half is None else [str(m._bias_half.dtype), bool(torch.equal(m._bias_half, m.bias.half()))],
                "buffers": sorted(m._buffers),
            }
    return {"layers": layers, "state_dict": {k: [str(v.dtype), list(v.shape)] for k, v in model.state_dict().items()}}


def main():
    sys.path.insert(0, str(ROOT))
    import oracle as O

    root = Path(sys.argv[1] if len(sys.argv) > 1 else "/root/reference")
    ql = load_by_path("_reference_quant_linear", root / "vdm_infer" / "quantization" / "quant_linear.py")
    pc = load_by_path("_reference_packed_checkpoint", root / "vdm_infer" / "checkpoints" / "packed_checkpoint.py")

    model = build_toy(ql.QuantLinear)
    for m in model.modules():
        if isinstance(m, ql.QuantLinear):
            m.set_quant_state(True, True)
    with torch.no_grad():
        model(torch.randn(16, 8))  # the quantizers take their scales: their buffers now sit in the state dict
    for m in model.modules():
        if isinstance(m, ql.QuantLinear):
            scale = m.wquantizer.scale.detach().view(-1)
            scale_h = scale.half()
            q = torch.clamp(torch.round(m.weight.detach() / scale_h.float()[:, None]), -8, 7).to(torch.int8).numpy()
            K = m.in_features
            m.register_buffer("vdm_weight_packed", torch.from_numpy(O.np_pack_wgt_v1(q)))
            m.register_buffer("vdm_weight_scale_packed", torch.from_numpy(O.np_pack_wscales_v1(scale_h.numpy(), K)))
            m.register_buffer("vdm_weight_scale", scale_h.clone())

    v1 = HERE / "reference_written_packed_v1.pt"
    pc.save_packed_checkpoint(model, str(v1), metadata={"written_by": "the reference's save_packed_checkpoint", "model": "toy 8-64-128-128"})
    payload = torch.load(str(v1), map_location="cpu", weights_only=True)
    legacy_sd = {}
    for k, v in payload["model"].items():
        for new, old in zip(pc.VDM_BUFFER_SUFFIXES, pc._LEGACY_BUFFER_SUFFIXES):
            if k.endswith("." + new):
                k = k[: -len(new)] + old
                break
        legacy_sd[k] = v
    legacy = HERE / "reference_written_packed_legacy.pt"
    torch.save({"format": pc._LEGACY_PACKED_CHECKPOINT_FORMAT, "metadata": payload["metadata"], "model": legacy_sd}, str(legacy))

    outcome = {"saved_keys": {k: [str(v.dtype), list(v.shape)] for k, v in payload["model"].items()}, "format": payload["format"],
               "metadata": payload["metadata"], "is_packed_checkpoint": {}, "loads": {}, "errors": {}}
    kw = dict(quant_linear_cls=ql.QuantLinear, dtype=torch.float16, device=torch.device("cpu"), require_vdm_kernel=False)
    for tag, path in (("v1", v1), ("legacy", legacy)):
        ckpt = pc.load_quant_checkpoint(str(path), dcp_loader=None)
        outcome["is_packed_checkpoint"][tag] = bool(pc.is_packed_checkpoint(ckpt))
        fresh = build_toy(ql.QuantLinear, seed=1)
        missing, unexpected = pc.load_packed_quantized_model(fresh, ckpt, **kw)
        entry = describe(fresh, ql.QuantLinear)
        entry["missing"], entry["unexpected"] = list(missing), list(unexpected)
        entry["re_export"] = {k: [str(v.dtype), list(v.shape)] for k, v in pc.packed_state_dict_from_model(fresh).items()}
        outcome["loads"][tag] = entry

    def error_of(fn):
        try:
            fn()
        except Exception as exc:  # the type and text are the record
            return [type(exc).__name__, str(exc)]
        return None

    broken = dict(payload, model={k: v for k, v in payload["model"].items() if k != "q2.vdm_weight_scale"})
    outcome["errors"]["missing_buffer"] = error_of(lambda: pc.load_packed_quantized_model(build_toy(ql.QuantLinear), broken, **kw))
    outcome["errors"]["other_format"] = error_of(lambda: pc.load_packed_quantized_model(build_toy(ql.QuantLinear), {"format": "other", "model": {}}, **kw))
    outcome["errors"]["not_a_dict"] = error_of(lambda: pc.load_packed_quantized_model(build_toy(ql.QuantLinear), [1, 2], **kw))
    plain = nn.Sequential(nn.Linear(4, 4))
    outcome["errors"]["no_quant_layers"] = error_of(
        lambda: pc.load_packed_quantized_model(plain, {"format": pc.PACKED_CHECKPOINT_FORMAT, "model": plain.state_dict()}, **kw))
    out = HERE / "reference_loader_outcome.json"
    out.write_text(json.dumps(outcome, indent=1, sort_keys=True) + "\n")
    for p in (v1, legacy, out):
        print(f"wrote {p} ({p.stat().st_size} bytes)")


if __name__ == "__main__":
    main()
