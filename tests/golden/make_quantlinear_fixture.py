#!/usr/bin/env python3
"""Writes tests/golden/quantlinear_fp_path.npz: input/output vectors of the reference's torch
floating-point path (UniformQuantizer, QuantLinear.forward without the kernel).

Nothing else pins that path bit for bit (the reference's tests hold no vectors for it), so this script
loads the reference's own vdm_infer/quantization/quant_linear.py -- that one file, by path, on the CPU --
and records what it computes on seeded inputs.  It runs only where the reference tree is present; the
tests read the committed .npz and never the reference.

    python tests/golden/make_quantlinear_fixture.py [/root/reference]
"""
import importlib.util
import sys
from pathlib import Path

import numpy as np
import torch
import torch.nn as nn


def load_reference(root: Path):
    # The reference tree is read-only by agreement: without this, the loader would leave a __pycache__ beside the file.
    sys.dont_write_bytecode = True
    spec = importlib.util.spec_from_file_location("_reference_quant_linear", root / "vdm_infer" / "quantization" / "quant_linear.py")
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


QUANTIZER_CASES = [
    # name, constructor arguments, input shape, input dtype
    ("sym_per_channel", dict(bit=4, sym=True), (24, 40), torch.float32),
    ("sym_clip", dict(bit=4, sym=True, clip_ratio=0.9), (24, 40), torch.float32),
    ("sym_per_token_3d", dict(bit=4, sym=True, granularity="per_token"), (3, 5, 32), torch.float32),
    ("sym_per_channel_3d", dict(bit=4, sym=True), (3, 5, 32), torch.float32),
    ("sym_per_tensor", dict(bit=8, sym=True, granularity="per_tensor"), (7, 16), torch.float32),
    ("sym_per_group", dict(bit=4, sym=True, granularity="per_group", group_size=8), (6, 32), torch.float32),
    ("asym_round_zero", dict(bit=4, sym=False), (12, 20), torch.float32),
    ("asym_no_round_zero", dict(bit=4, sym=False, round_zero=False), (12, 20), torch.float32),
    ("sym_fp16", dict(bit=4, sym=True), (16, 64), torch.float16),
]


def main():
    root = Path(sys.argv[1] if len(sys.argv) > 1 else "/root/reference")
    ref = load_reference(root)
    torch.manual_seed(20240611)
    out = {}
    for name, kw, shape, dtype in QUANTIZER_CASES:
        x = torch.randn(shape).to(dtype)
        x.view(-1)[3] *= 9.0  # an outlier
        q = ref.UniformQuantizer(**kw)
        y = q(x)
        x2 = (torch.randn(shape) * 3.0).to(dtype)  # the parameters are frozen after the first tensor
        y2 = q(x2)
        out[f"q.{name}.x"], out[f"q.{name}.y"] = x.numpy(), y.numpy()
        out[f"q.{name}.x2"], out[f"q.{name}.y2"] = x2.numpy(), y2.numpy()
        out[f"q.{name}.scale"] = q.scale.numpy()
        if q.zero_point is not None:
            out[f"q.{name}.zero_point"] = q.zero_point.numpy()

    qp = {"w": {"bit": 4, "sym": True}, "act": {"bit": 4, "sym": True}}
    for name, bias, xshape in (("bias_2d", True, (16, 40)), ("nobias_2d", False, (16, 40)), ("bias_3d", True, (2, 9, 40))):
        layer = nn.Linear(40, 24, bias=bias)
        m = ref.QuantLinear(layer, {"w": "lsq", "act": "dynamic"}, qp)
        x = torch.randn(xshape)
        x.view(-1, 40)[:, 7] *= 20.0
        x2 = torch.randn(xshape) * 2.0
        with torch.no_grad():
            plain = m(x)
            m.set_quant_state(True, False)
            w_only = m(x)
            m.set_quant_state(True, True)
            both = m(x)
            both2 = m(x2)  # activation scale frozen by the call before
        out[f"l.{name}.weight"] = layer.weight.detach().numpy()
        if bias:
            out[f"l.{name}.bias"] = layer.bias.detach().numpy()
        out[f"l.{name}.x"], out[f"l.{name}.x2"] = x.numpy(), x2.numpy()
        out[f"l.{name}.plain"], out[f"l.{name}.w_only"] = plain.numpy(), w_only.numpy()
        out[f"l.{name}.both"], out[f"l.{name}.both2"] = both.numpy(), both2.numpy()
        out[f"l.{name}.wscale"], out[f"l.{name}.ascale"] = m.wquantizer.scale.numpy(), m.aquantizer.scale.numpy()
        out[f"l.{name}.repr"] = np.array(m.extra_repr())
    path = Path(__file__).with_name("quantlinear_fp_path.npz")
    np.savez_compressed(path, **out)
    print(f"wrote {path} ({path.stat().st_size} bytes, {len(out)} arrays)")


if __name__ == "__main__":
    main()
