"""The two listings of INTEGRATION.md that show how a maintainer of the reference binds the C ABI from the reference's
own wrapper (sections B and D) are executed as they stand in the document and held to the oracle: documentation that
no longer matches the library fails here."""
import re
from pathlib import Path

import numpy as np
import pytest
import torch

import oracle as O

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
ROOT = Path(__file__).resolve().parent.parent


def _listings():
    text = (ROOT / "INTEGRATION.md").read_text()
    blocks = re.findall(r"```python\n(.*?)```", text, flags=re.S)
    binding = [b for b in blocks if "def linear_vdm_w4a4(" in b]
    fast = [b for b in blocks if "def linear_vdm_w4a4_fast(" in b]
    assert len(binding) == 1 and len(fast) == 1
    return binding[0], fast[0]


def test_documented_bindings_run_and_match_the_oracle():
    from dsaquant_amd import _lib
    from dsaquant_amd.kernels import vdm_w4a4 as v

    assert v.is_available(), v.load_error()
    binding, fast = _listings()
    # the listing loads "libvdmq.so" by name; here it is the library built in this tree
    binding = binding.replace('ctypes.CDLL("libvdmq.so")', f'ctypes.CDLL("{_lib.LIB_PATH}")')
    assert str(_lib.LIB_PATH) in binding

    # the two helpers of the reference's wrapper that the listing leaves unchanged (vdm_w4a4.py:182-184, 198-206)
    def _as_2d_half_contiguous(x):
        return x.reshape(-1, x.shape[-1]).half().contiguous(), tuple(x.shape[:-1])

    def _check_linear_shapes(x_2d, qweight, wscales):
        if qweight.shape[1] * 2 != x_2d.shape[1] or wscales.shape[0] != qweight.shape[0]:
            raise ValueError("shape mismatch")

    ns = {"_as_2d_half_contiguous": _as_2d_half_contiguous, "_check_linear_shapes": _check_linear_shapes}
    exec(compile(binding, "INTEGRATION.md section B", "exec"), ns)
    exec(compile(fast, "INTEGRATION.md section D", "exec"), ns)

    for M, K, N in ((300, 1536, 384), (515, 256, 256), (4100, 1536, 4608)):
        x, qw, ws, bias = O.synth_linear(M, K, N, seed=M)
        xt = torch.from_numpy(x).to(DEV).view(1, M, K)
        qv1 = torch.from_numpy(O.np_pack_wgt_v1(qw)).to(DEV)
        sv1 = torch.from_numpy(O.np_pack_wscales_v1(ws, K)).to(DEV)
        bt = torch.from_numpy(bias).to(DEV)
        want = O.np_linear(x, qw, ws, bias, 1.0)[0]
        for name in ("linear_vdm_w4a4", "linear_vdm_w4a4_fast"):
            print(f"documented binding {name} M={M} K={K} N={N}", flush=True)
            got = ns[name](xt, qv1, sv1, bt, clip_ratio=1.0)
            torch.cuda.synchronize()
            assert got.shape == (1, M, N) and got.dtype == torch.float16
            assert np.array_equal(got.view(M, N).cpu().numpy().view(np.uint16), want.view(np.uint16)), (name, M, K, N)
        assert bool(ns["_L"].vdmq_bf6_pays(M, N, K)) == (K >= 1280)
