"""ctypes binding of libvdmq.so (the C ABI in include/vdmq.h)."""
from __future__ import annotations

import ctypes
import os
import subprocess
from pathlib import Path
from typing import Optional

_PKG = Path(__file__).resolve().parent
LIB_PATH = _PKG / "libvdmq.so"
CSRC = _PKG / "csrc"

_LIB: Optional[ctypes.CDLL] = None

VDMQ_VERSION = 2  # include/vdmq.h; also the version of the bf6 block format
VDMQ_OUT_F16 = 0
VDMQ_OUT_BF16 = 1
VDMQ_ACT_NONE = 0
VDMQ_ACT_GELU_TANH = 1
VDMQ_LN_MODULATE = 1
VDMQ_LN_AFFINE = 2

class GemmLaunchInfo(ctypes.Structure):
    """vdmq_gemm_launch_info of include/vdmq.h."""
    _fields_ = [("kernel", ctypes.c_int), ("tile_m", ctypes.c_int), ("tile_n", ctypes.c_int), ("group_m", ctypes.c_int),
                ("group_n", ctypes.c_int), ("contiguous_runs", ctypes.c_int), ("workgroups", ctypes.c_int64)]


KERNEL_GEMM_W4A4, KERNEL_GEMM_BF6, KERNEL_GEMM_BF6_PERSISTENT = 1, 2, 3

# name -> (restype, argtypes); every symbol include/vdmq.h declares
_i64, _p, _f32, _int = ctypes.c_int64, ctypes.c_void_p, ctypes.c_float, ctypes.c_int
SIGNATURES = {
    "vdmq_version": (_int, []),
    "vdmq_arch": (ctypes.c_char_p, []),
    "vdmq_last_error": (ctypes.c_char_p, []),
    "vdmq_k_padded": (_i64, [_i64]),
    "vdmq_quantize_act": (_int, [_p, _i64, _i64, _i64, _f32, _p, _p, _p]),
    "vdmq_quantize_act_ex": (_int, [_p, _i64, _i64, _i64, _f32, _int, _p, _p, _p]),
    "vdmq_quantize_act_ln": (_int, [_p, _i64, _i64, _i64, _f32, _int, _p, _p, _i64, _i64, _f32, _p, _p, _p]),
    "vdmq_ln_f16": (_int, [_p, _i64, _i64, _i64, _f32, _int, _p, _p, _i64, _i64, _p, _i64, _p]),
    "vdmq_linear_ln_w4a4": (_int, [_p, _i64, _i64, _i64, _f32, _int, _p, _p, _i64, _i64, _f32, _p, _p, _p, _p, _int, _i64, _i64, _p, _i64, _p]),
    "vdmq_gelu_tanh_f16": (_int, [_p, _p, _i64, _p]),
    "vdmq_gemm_w4a4": (_int, [_p, _p, _p, _p, _p, _p, _int, _i64, _i64, _i64, _i64, _p]),
    "vdmq_gemm_w4a4_ex": (_int, [_p, _p, _p, _p, _p, _p, _i64, _i64, _p, _i64, _p, _int, _i64, _i64, _i64, _i64, _p]),
    "vdmq_gemm_w4a4_acc": (_int, [_p, _p, _p, _i64, _i64, _i64, _p]),
    "vdmq_gemm_w4a4_split": (_int, [_p, _p, _p, _p, _p, _p, _i64, _i64, _i64, _i64, _i64, _i64, _p]),
    "vdmq_gemm_w4a4_bf6_split": (_int, [_p, _p, _p, _p, _p, _p, _i64, _i64, _i64, _i64, _i64, _i64, _p]),
    "vdmq_last_gemm_launch": (_int, [ctypes.POINTER(GemmLaunchInfo)]),
    "vdmq_workspace_bytes": (_i64, [_i64, _i64]),
    "vdmq_linear_w4a4": (_int, [_p, _i64, _i64, _i64, _f32, _p, _p, _p, _p, _int, _i64, _i64, _p, _i64, _p]),
    "vdmq_linear_w4a4_ex": (_int, [_p, _i64, _i64, _i64, _f32, _int, _p, _p, _p, _p, _int, _i64, _i64, _p, _i64, _p]),
    "vdmq_linear_w4a4_noalloc": (_int, [_p, _i64, _i64, _i64, _f32, _p, _p, _p, _p, _int, _i64, _i64, _p]),
    "vdmq_weight_v1_to_native": (_int, [_p, _p, _i64, _i64, _p]),
    "vdmq_weight_native_to_v1": (_int, [_p, _p, _i64, _i64, _p]),
    "vdmq_wscale_v1_to_plain": (_int, [_p, _p, _i64, _i64, _p]),
    "vdmq_wscale_plain_to_v1": (_int, [_p, _p, _i64, _i64, _p]),
    "vdmq_act_native_to_v1": (_int, [_p, _p, _i64, _i64, _p, _p, _p]),
    "vdmq_act_v1_to_native": (_int, [_p, _p, _i64, _i64, _p, _p, _p]),
    "vdmq_row_scale": (_int, [_p, _i64, _i64, _f32, _p, _p]),
    "vdmq_quantize_weight_native": (_int, [_p, _p, _p, _i64, _i64, _p]),
    "vdmq_bf6_bytes": (_i64, [_i64, _i64]),
    "vdmq_quantize_act_bf6": (_int, [_p, _i64, _i64, _i64, _f32, _int, _p, _p, _p]),
    "vdmq_quantize_act_ln_bf6": (_int, [_p, _i64, _i64, _i64, _f32, _int, _p, _p, _i64, _i64, _f32, _p, _p, _p]),
    "vdmq_workspace_bytes_bf6": (_i64, [_i64, _i64]),
    "vdmq_bf6_pays": (_int, [_i64, _i64, _i64]),
    "vdmq_linear_w4a4_bf6": (_int, [_p, _i64, _i64, _i64, _f32, _int, _p, _p, _p, _p, _int, _i64, _i64, _p, _i64, _p]),
    "vdmq_native_to_bf6": (_int, [_p, _i64, _i64, _p, _p]),
    "vdmq_weight_v1_to_bf6": (_int, [_p, _p, _i64, _i64, _p]),
    "vdmq_bf6_to_weight_v1": (_int, [_p, _p, _i64, _i64, _p]),
    "vdmq_gemm_w4a4_bf6": (_int, [_p, _p, _p, _p, _p, _p, _int, _i64, _i64, _i64, _i64, _p]),
    "vdmq_gemm_w4a4_bf6_ex": (_int, [_p, _p, _p, _p, _p, _p, _i64, _i64, _p, _i64, _p, _int, _i64, _i64, _i64, _i64, _p]),
    "vdmq_gemm_w4a4_bf6_acc": (_int, [_p, _p, _p, _i64, _i64, _i64, _p]),
    "vdmq_copy_u128": (_int, [_p, _p, _i64, _p]),
    "vdmq_stream_probe": (_int, [_p, _p, _i64, _int, _int, _p]),
    "vdmq_mfma_probe_operand_bytes": (_i64, []),
    "vdmq_mfma_probe": (_int, [_int, _p, _i64, _i64, _p, ctypes.POINTER(ctypes.c_double), _p]),
}


class VdmqError(RuntimeError):
    """A native precondition failed (the reference raises RuntimeError from TORCH_CHECK)."""


def build(verbose: bool = False) -> Path:
    """Compile libvdmq.so for gfx950 with hipcc (``make -C dsaquant_amd/csrc``)."""
    cmd = ["make", "-C", str(CSRC), "-j", str(min(8, os.cpu_count() or 1)), "-B"]
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if verbose or res.returncode != 0:
        print(res.stdout)
    if res.returncode != 0:
        raise RuntimeError("building libvdmq.so failed")
    return LIB_PATH


def load() -> ctypes.CDLL:
    """Load the built library; raises if it is missing (no fallback exists)."""
    global _LIB
    if _LIB is not None:
        return _LIB
    if not LIB_PATH.exists():
        raise FileNotFoundError(
            f"{LIB_PATH} is missing: build it with `python -c 'import __graft_entry__ as g; g.build()'` "
            f"or `make -C {CSRC}`")
    lib = ctypes.CDLL(str(LIB_PATH))
    for name, (restype, argtypes) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = restype
        fn.argtypes = argtypes
    if lib.vdmq_version() != VDMQ_VERSION:
        raise RuntimeError(f"{LIB_PATH} has interface version {lib.vdmq_version()}, this package expects {VDMQ_VERSION}: rebuild it (make -C {CSRC})")
    _LIB = lib
    return lib


def last_gemm_launch() -> GemmLaunchInfo:
    """What the library chose for the last GEMM launched on this thread."""
    info = GemmLaunchInfo()
    check(load().vdmq_last_gemm_launch(ctypes.byref(info)))
    return info


def check(rc: int) -> None:
    if rc != 0:
        msg = load().vdmq_last_error()
        raise VdmqError(f"vdmq error {rc}: {msg.decode() if msg else ''}")
