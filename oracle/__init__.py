"""CPU oracle for the W4A4 linear hot path -- TEST INFRASTRUCTURE ONLY.

Only tests, the smoke check and the benchmark's CPU-baseline leg may import
this package.  The product (``dsaquant_amd``) never does.

Two layers, pinned against each other by ``tests/test_oracle.py``:

* ``c_*``  -- thin ctypes wrappers over ``vdmq_oracle.c``, the scalar C
  restatement of ``vdm_infer/kernels/csrc/vdm_w4a4_kernel.cu`` (each C
  function cites the lines it follows).
* ``np_*`` -- vectorised numpy forms of the same closed formulas, fast enough
  for the larger parity shapes.

All arrays are numpy.  fp16 data is ``np.float16``; quantized values in the
logical domain are ``np.int8`` holding int4 values; packed buffers are
``np.uint8``.
"""
from __future__ import annotations

import ctypes
import os
import subprocess
from pathlib import Path

import numpy as np

_HERE = Path(__file__).resolve().parent
_LIB_PATH = _HERE / "_build" / "libvdmq_oracle.so"
_LIB = None

BLOCK_M = 256
BLOCK_N = 128
WARP_K = 64


def build(force: bool = False) -> Path:
    """Compile vdmq_oracle.c with gcc (``make -C oracle``)."""
    if force or not _LIB_PATH.exists() or _LIB_PATH.stat().st_mtime < (_HERE / "vdmq_oracle.c").stat().st_mtime:
        subprocess.run(["make", "-C", str(_HERE), "-B" if force else "-s"], check=True, stdout=subprocess.DEVNULL)
    return _LIB_PATH


def lib() -> ctypes.CDLL:
    global _LIB
    if _LIB is None:
        build()
        L = ctypes.CDLL(str(_LIB_PATH))
        i64, p, f32 = ctypes.c_int64, ctypes.c_void_p, ctypes.c_float
        L.vdmq_oracle_h2f.restype = ctypes.c_float
        L.vdmq_oracle_h2f.argtypes = [ctypes.c_uint16]
        L.vdmq_oracle_f2h.restype = ctypes.c_uint16
        L.vdmq_oracle_f2h.argtypes = [ctypes.c_float]
        L.vdmq_oracle_d2h.restype = ctypes.c_uint16
        L.vdmq_oracle_d2h.argtypes = [ctypes.c_double]
        L.vdmq_oracle_row_scale.argtypes = [p, i64, i64, f32, p]
        L.vdmq_oracle_quantize_rows.argtypes = [p, p, i64, i64, p]
        for name in ("act", "wgt"):
            fn = getattr(L, f"vdmq_oracle_{name}_v1_offset")
            fn.restype = i64
            fn.argtypes = [i64, i64, i64, ctypes.POINTER(ctypes.c_int)]
        for name in ("ascale", "wscale"):
            fn = getattr(L, f"vdmq_oracle_{name}_v1_index")
            fn.restype = i64
            fn.argtypes = [i64, i64, i64]
        for name in ("pack_act_v1", "unpack_act_v1", "pack_ascales_v1", "pack_wgt_v1", "unpack_wgt_v1",
                     "pack_wscales_v1", "unpack_wscales_v1"):
            getattr(L, f"vdmq_oracle_{name}").argtypes = [p, i64, i64, p]
        L.vdmq_oracle_gemm_i32.argtypes = [p, p, i64, i64, i64, p]
        L.vdmq_oracle_epilogue.argtypes = [p, p, p, p, i64, i64, p]
        L.vdmq_oracle_linear.argtypes = [p, p, p, p, f32, i64, i64, i64, p, p, p, p]
        _LIB = L
    return _LIB


def _ptr(a: np.ndarray):
    assert a.flags["C_CONTIGUOUS"]
    return a.ctypes.data_as(ctypes.c_void_p)


def _c(a, dtype) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=dtype)


def padded_m(M: int) -> int:
    return (M + BLOCK_M - 1) // BLOCK_M * BLOCK_M


# ---------------------------------------------------------------- C wrappers

def c_row_scale(x: np.ndarray, clip: float = 1.0) -> np.ndarray:
    x = _c(x, np.float16)
    M, K = x.shape
    out = np.empty(M, np.float16)
    lib().vdmq_oracle_row_scale(_ptr(x), M, K, clip, _ptr(out))
    return out


def c_quantize_rows(x: np.ndarray, scale_h: np.ndarray) -> np.ndarray:
    x = _c(x, np.float16)
    scale_h = _c(scale_h, np.float16)
    M, K = x.shape
    q = np.empty((M, K), np.int8)
    lib().vdmq_oracle_quantize_rows(_ptr(x), _ptr(scale_h), M, K, _ptr(q))
    return q


def c_pack_act_v1(q: np.ndarray) -> np.ndarray:
    q = _c(q, np.int8)
    M, K = q.shape
    out = np.empty((padded_m(M), K // 2), np.uint8)
    lib().vdmq_oracle_pack_act_v1(_ptr(q), M, K, _ptr(out))
    return out


def c_unpack_act_v1(qact: np.ndarray, M: int, K: int) -> np.ndarray:
    qact = _c(qact, np.uint8)
    q = np.empty((M, K), np.int8)
    lib().vdmq_oracle_unpack_act_v1(_ptr(qact), M, K, _ptr(q))
    return q


def c_pack_ascales_v1(scale_h: np.ndarray, K: int) -> np.ndarray:
    scale_h = _c(scale_h, np.float16)
    M = scale_h.shape[0]
    out = np.empty((padded_m(M), K // WARP_K), np.float16)
    lib().vdmq_oracle_pack_ascales_v1(_ptr(scale_h), M, K, _ptr(out))
    return out


def c_pack_wgt_v1(q: np.ndarray) -> np.ndarray:
    q = _c(q, np.int8)
    N, K = q.shape
    out = np.empty((N, K // 2), np.uint8)
    lib().vdmq_oracle_pack_wgt_v1(_ptr(q), N, K, _ptr(out))
    return out


def c_unpack_wgt_v1(qweight: np.ndarray, N: int, K: int) -> np.ndarray:
    qweight = _c(qweight, np.uint8)
    q = np.empty((N, K), np.int8)
    lib().vdmq_oracle_unpack_wgt_v1(_ptr(qweight), N, K, _ptr(q))
    return q


def c_pack_wscales_v1(scale_h: np.ndarray, K: int) -> np.ndarray:
    scale_h = _c(scale_h, np.float16)
    N = scale_h.shape[0]
    out = np.empty((N, K // WARP_K), np.float16)
    lib().vdmq_oracle_pack_wscales_v1(_ptr(scale_h), N, K, _ptr(out))
    return out


def c_unpack_wscales_v1(packed: np.ndarray, N: int, K: int) -> np.ndarray:
    packed = _c(packed, np.float16)
    out = np.empty(N, np.float16)
    lib().vdmq_oracle_unpack_wscales_v1(_ptr(packed), N, K, _ptr(out))
    return out


def c_gemm_i32(qx: np.ndarray, qw: np.ndarray) -> np.ndarray:
    qx, qw = _c(qx, np.int8), _c(qw, np.int8)
    M, K = qx.shape
    N = qw.shape[0]
    acc = np.empty((M, N), np.int32)
    lib().vdmq_oracle_gemm_i32(_ptr(qx), _ptr(qw), M, N, K, _ptr(acc))
    return acc


def c_epilogue(acc, as_h, ws_h, bias_h=None) -> np.ndarray:
    acc = _c(acc, np.int32)
    as_h, ws_h = _c(as_h, np.float16), _c(ws_h, np.float16)
    M, N = acc.shape
    out = np.empty((M, N), np.float16)
    b = None if bias_h is None else _c(bias_h, np.float16)
    lib().vdmq_oracle_epilogue(_ptr(acc), _ptr(as_h), _ptr(ws_h), None if b is None else _ptr(b), M, N, _ptr(out))
    return out


def c_linear(x, qw, ws_h, bias_h=None, clip: float = 1.0):
    """Whole path in scalar C.  Returns (out, qx, as_h, acc)."""
    x = _c(x, np.float16)
    qw = _c(qw, np.int8)
    ws_h = _c(ws_h, np.float16)
    M, K = x.shape
    N = qw.shape[0]
    qx = np.empty((M, K), np.int8)
    as_h = np.empty(M, np.float16)
    acc = np.empty((M, N), np.int32)
    out = np.empty((M, N), np.float16)
    b = None if bias_h is None else _c(bias_h, np.float16)
    lib().vdmq_oracle_linear(_ptr(x), _ptr(qw), _ptr(ws_h), None if b is None else _ptr(b), clip, M, N, K, _ptr(qx),
                             _ptr(as_h), _ptr(acc), _ptr(out))
    return out, qx, as_h, acc


# ------------------------------------------------------------- numpy forms

def np_gelu_tanh_f64(x) -> np.ndarray:
    """GELU, tanh approximation, in float64.  The reference's FFN is diffusers'
    FeedForward(activation_fn="gelu-approximate") (dit_block.py:56), i.e. torch's
    GELU(approximate="tanh"), whose published definition is
        0.5 * x * (1 + tanh(sqrt(2/pi) * (x + 0.044715 * x^3))).
    0.5 * (1 + tanh(u)) is written as 1 / (1 + exp(-2u)) (the same function, without
    the cancellation of 1 + tanh(u) for very negative u)."""
    x = np.asarray(x, dtype=np.float64)
    with np.errstate(over="ignore", invalid="ignore"):
        u = np.sqrt(2.0 / np.pi) * (x + 0.044715 * x * x * x)
        return x / (1.0 + np.exp(-2.0 * u))


def np_gelu_tanh_f16(x_h: np.ndarray) -> np.ndarray:
    """The correctly rounded fp16 GELU of fp16 inputs: what a framework's fp32
    evaluation on an fp16 tensor approximates (one rounding to fp16)."""
    assert x_h.dtype == np.float16
    with np.errstate(over="ignore", invalid="ignore"):
        return np_gelu_tanh_f64(x_h).astype(np.float16)


def np_layer_norm_f64(x_h: np.ndarray, eps: float) -> np.ndarray:
    """LayerNorm without affine over the last axis, float64: (x - mean) / sqrt(var + eps), biased variance
    (FP32LayerNorm of the reference's blocks, dit_block.py:32,56: torch.nn.functional.layer_norm on x.float())."""
    x = x_h.astype(np.float64)
    mean = x.mean(axis=-1, keepdims=True)
    var = ((x - mean) ** 2).mean(axis=-1, keepdims=True)
    return (x - mean) / np.sqrt(var + eps)


def np_ln_modulate_f16(x_h: np.ndarray, scale_h: np.ndarray, shift_h: np.ndarray, eps: float, rows_per_vec: int = 1):
    """norm(x) * (1 + scale) + shift as the reference evaluates it on fp16 tensors (dit_block.py:100, :110): the
    LayerNorm result is cast to fp16, then three fp16 tensor operations, each correctly rounded.  Returns
    (h, aux) with aux = the intermediate fp16 tensors ln, s1 = 1 + scale and p = ln * s1 (an error bound for an
    implementation whose LayerNorm is one ulp off needs their magnitudes)."""
    ln = np_layer_norm_f64(x_h, eps).astype(np.float16)
    a = np.repeat(scale_h.reshape(-1, x_h.shape[-1]), rows_per_vec, axis=0)
    b = np.repeat(shift_h.reshape(-1, x_h.shape[-1]), rows_per_vec, axis=0)
    s1 = (np.float16(1.0) + a).astype(np.float16)
    p = (ln.astype(np.float32) * s1.astype(np.float32)).astype(np.float16)  # product of two fp16 is exact in fp32
    h = (p.astype(np.float64) + b.astype(np.float64)).astype(np.float16)     # exact sum, one rounding
    return h, {"ln": ln, "s1": s1, "p": p}


def np_ln_affine_f16(x_h: np.ndarray, weight_h: np.ndarray, bias_h: np.ndarray, eps: float, rows_per_vec: int = 1) -> np.ndarray:
    """FP32LayerNorm with elementwise affine (norm2, dit_block.py:53): LN(x) * w + b, one rounding to fp16."""
    a = np.repeat(weight_h.reshape(-1, x_h.shape[-1]), rows_per_vec, axis=0).astype(np.float64)
    b = np.repeat(bias_h.reshape(-1, x_h.shape[-1]), rows_per_vec, axis=0).astype(np.float64)
    return (np_layer_norm_f64(x_h, eps) * a + b).astype(np.float16)


def np_row_scale(x: np.ndarray, clip: float = 1.0) -> np.ndarray:
    """vdm_w4a4_kernel.cu:459-481 -- fp32 absmax ignoring NaN, /7, *clip, fp16."""
    a = np.abs(x.astype(np.float32))
    with np.errstate(invalid="ignore"):
        mx = np.fmax.reduce(a, axis=1, initial=np.float32(0.0))  # fmax ignores NaN
    with np.errstate(over="ignore", invalid="ignore"):
        s = np.where(mx > 0, (mx / np.float32(7.0)) * np.float32(clip), np.float32(1.0)).astype(np.float32)
        return s.astype(np.float16)


def np_quantize_rows(x: np.ndarray, scale_h: np.ndarray) -> np.ndarray:
    """vdm_w4a4_kernel.cu:95-102, 319-329 -- reciprocal multiply, rni, sat s4."""
    with np.errstate(divide="ignore", invalid="ignore", over="ignore"):
        rscale = (np.float32(1.0) / scale_h.astype(np.float32)).astype(np.float32)
        v = x.astype(np.float32) * rscale[:, None]
        r = np.rint(v)  # round half to even
        r = np.where(np.isnan(r), np.float32(0), r)
        return np.clip(r, -8, 7).astype(np.int8)


def np_gemm_i32(qx: np.ndarray, qw: np.ndarray) -> np.ndarray:
    """Exact integer matmul through fp32 BLAS: every partial sum is an integer
    of magnitude <= 64*K < 2**24, so fp32 accumulation is exact."""
    K = qx.shape[1]
    assert 64 * K < (1 << 24)
    return (qx.astype(np.float32) @ qw.astype(np.float32).T).astype(np.int32)


def np_epilogue(acc, as_h, ws_h, bias_h=None) -> np.ndarray:
    """vdm_w4a4_kernel.cu:243-274, 557-569."""
    s = as_h.astype(np.float32)[:, None] * ws_h.astype(np.float32)[None, :]
    with np.errstate(over="ignore", invalid="ignore"):
        h = (acc.astype(np.float32) * s).astype(np.float16)
        if bias_h is not None:
            # exact sum of two fp16 values in float64, one rounding to fp16
            h = (h.astype(np.float64) + bias_h.astype(np.float64)[None, :]).astype(np.float16)
    return h


def np_gated_residual(y_h: np.ndarray, gate_h, res_h, rows_per_gate: int = 1) -> np.ndarray:
    """hidden_states + attn_output * gate on fp16 tensors (dit_block.py:102, :107, :112): the product rounded to
    fp16, then the sum rounded to fp16.  gate_h [*, N] (row m uses row m // rows_per_gate) or None; res_h or None."""
    out = y_h
    if gate_h is not None:
        g = np.repeat(gate_h.reshape(-1, y_h.shape[-1]), rows_per_gate, axis=0)
        with np.errstate(over="ignore", invalid="ignore"):
            out = (out.astype(np.float32) * g.astype(np.float32)).astype(np.float16)  # exact product, one rounding
    if res_h is not None:
        with np.errstate(over="ignore", invalid="ignore"):
            out = (res_h.astype(np.float64) + out.astype(np.float64)).astype(np.float16)  # exact sum, one rounding
    return out


# E3M2 ("bf6") codes: sign << 5 | exponent << 2 | mantissa, value = 2^(e-3) * (1 + m/4) for e > 0 and m / 16 for
# e = 0 (OCP Microscaling Formats specification, FP6 E3M2, bias 3; no infinities or NaNs).  The operand blocks hold
# an int4 value q as the E3M2 float q / 16, whose code is sign << 5 | |q|.
BF6_BLOCK_SCALE = 16.0
def np_bf6_decode(code: np.ndarray) -> np.ndarray:
    """E3M2 code (0..63) -> value, straight from the format definition (subnormals included)."""
    code = code.astype(np.int64)
    sign = np.where(code & 32, -1.0, 1.0)
    e, m = (code >> 2) & 7, code & 3
    mag = np.where(e == 0, m / 4.0 * 2.0 ** -2, 2.0 ** (e - 3.0) * (1.0 + m / 4.0))
    return sign * mag


def np_unpack_bf6_blocks(blocks: np.ndarray, rows: int, K: int) -> np.ndarray:
    """bf6 operand buffer (u8) -> the integers it stands for, float64 [rows, K] (E3M2 value x 16).  Layout: rows padded to 32 and stored in panels of 8, K padded
    to 128 and cut into k-blocks of 64; a panel holds its k-blocks one after the other, 384 bytes each =
    [h = 0: 8 rows x 16 B][h = 1: 8 rows x 16 B][h = 0: 8 rows x 8 B][h = 1: 8 rows x 8 B].  A row's 16-byte and 8-byte
    parts for (k-block, h) form one 192-bit little-endian string holding the 32 six-bit codes of k = 64 kb + 32 h + e
    (code e at bits 6e..6e+5) -- the operand registers of lane (row % 32) + 32 h of v_mfma_f32_32x32x64_f8f6f4.
    Also checks the zero padding."""
    kblocks = (K + 127) // 128 * 2
    panels = (rows + 31) // 32 * 4
    b = blocks.reshape(panels, kblocks, 384)
    lo = b[:, :, :256].reshape(panels, kblocks, 2, 8, 16)
    hi = b[:, :, 256:].reshape(panels, kblocks, 2, 8, 8)
    s = np.concatenate([lo, hi], axis=4)                      # [panel, kb, h, row in panel, 24 bytes]
    bits = np.unpackbits(s, axis=4, bitorder="little")        # 192 bits
    codes = (bits.reshape(panels, kblocks, 2, 8, 32, 6) * (1 << np.arange(6))).sum(axis=5)
    vals = np_bf6_decode(codes) * BF6_BLOCK_SCALE             # [panel, kb, h, j, e]
    full = vals.transpose(0, 3, 1, 2, 4).reshape(panels * 8, kblocks * 64)
    assert not full[rows:].any() and not full[:, K:].any(), "padding must be zero"
    return full[:rows, :K]


def np_linear(x, qw, ws_h, bias_h=None, clip: float = 1.0):
    as_h = np_row_scale(x, clip)
    qx = np_quantize_rows(x, as_h)
    acc = np_gemm_i32(qx, qw)
    return np_epilogue(acc, as_h, ws_h, bias_h), qx, as_h, acc


# v1 layout index arrays (vectorised restatement of the offset formulas in
# vdmq_oracle.c; pinned against the C functions element by element in tests)

def np_act_v1_offsets(M: int, K: int):
    m = np.arange(M, dtype=np.int64)[:, None]
    k = np.arange(K, dtype=np.int64)[None, :]
    KG = K // WARP_K
    bm, warp, tile, r = m // BLOCK_M, (m % BLOCK_M) // 32, (m % 32) // 16, m % 16
    g, hi_m = r % 8, r // 8
    bk, kk = k // WARP_K, k % WARP_K
    c = kk // 8
    khalf, t = c // 4, c % 4
    lane, comp = 4 * g + t, 2 * khalf + hi_m
    off = (((((bm * KG + bk) * 8 + warp) * 2 + tile) * 32 + lane) * 16) + 4 * comp + (kk % 8) // 2
    return off, np.broadcast_to(kk & 1, off.shape)


def np_wgt_v1_offsets(N: int, K: int):
    n = np.arange(N, dtype=np.int64)[:, None]
    k = np.arange(K, dtype=np.int64)[None, :]
    KG = K // WARP_K
    bn, tile, r = n // BLOCK_N, (n % BLOCK_N) // 16, n % 16
    g, hi_n = r % 8, r // 8
    bk, kk = k // WARP_K, k % WARP_K
    c = kk // 8
    khalf, t = c // 4, c % 4
    lane, comp = 4 * g + t, 2 * hi_n + khalf
    off = ((((bn * KG + bk) * 8 + tile) * 32 + lane) * 16) + 4 * comp + (kk % 8) // 2
    return off, np.broadcast_to(kk & 1, off.shape)


def _np_pack(q: np.ndarray, off: np.ndarray, hi: np.ndarray, nbytes: int) -> np.ndarray:
    buf = np.zeros(nbytes, np.uint8)
    v = (q.astype(np.uint8) & 0xF)
    lo = hi == 0
    buf[off[lo]] |= v[lo]
    buf[off[~lo]] |= (v[~lo] << 4).astype(np.uint8)
    return buf


def _np_unpack(buf: np.ndarray, off: np.ndarray, hi: np.ndarray) -> np.ndarray:
    b = buf.reshape(-1)[off]
    v = np.where(hi == 0, b & 0xF, b >> 4).astype(np.int8)
    return np.where(v >= 8, v - 16, v).astype(np.int8)


def np_pack_act_v1(q: np.ndarray) -> np.ndarray:
    M, K = q.shape
    off, hi = np_act_v1_offsets(M, K)
    return _np_pack(q, off, hi, padded_m(M) * K // 2).reshape(padded_m(M), K // 2)


def np_unpack_act_v1(qact: np.ndarray, M: int, K: int) -> np.ndarray:
    off, hi = np_act_v1_offsets(M, K)
    return _np_unpack(qact, off, hi)


def np_pack_wgt_v1(q: np.ndarray) -> np.ndarray:
    N, K = q.shape
    off, hi = np_wgt_v1_offsets(N, K)
    return _np_pack(q, off, hi, N * K // 2).reshape(N, K // 2)


def np_unpack_wgt_v1(qweight: np.ndarray, N: int, K: int) -> np.ndarray:
    off, hi = np_wgt_v1_offsets(N, K)
    return _np_unpack(qweight, off, hi)


def np_wscale_v1_indices(N: int, K: int) -> np.ndarray:
    n = np.arange(N, dtype=np.int64)[:, None]
    bk = np.arange(K // WARP_K, dtype=np.int64)[None, :]
    KG = K // WARP_K
    bn, j, r = n // BLOCK_N, (n % BLOCK_N) // 16, n % 16
    return (((bn * KG + bk) * 32 + 4 * j + (r % 8) // 2) * 4) + 2 * (r // 8) + r % 2


def np_ascale_v1_indices(PM: int, K: int) -> np.ndarray:
    m = np.arange(PM, dtype=np.int64)[:, None]
    bk = np.arange(K // WARP_K, dtype=np.int64)[None, :]
    KG = K // WARP_K
    bm, warp, i, r = m // BLOCK_M, (m % BLOCK_M) // 32, (m % 32) // 16, m % 16
    return ((((bm * KG + bk) * 8 + warp) * 16 + 8 * i + r % 8) * 2) + r // 8


def np_pack_wscales_v1(scale_h: np.ndarray, K: int) -> np.ndarray:
    N = scale_h.shape[0]
    idx = np_wscale_v1_indices(N, K)
    out = np.empty(N * (K // WARP_K), np.float16)
    out[idx] = scale_h[:, None]
    return out.reshape(N, K // WARP_K)


def np_unpack_wscales_v1(packed: np.ndarray, N: int, K: int) -> np.ndarray:
    return packed.reshape(-1)[np_wscale_v1_indices(N, K)[:, 0]]


def np_pack_ascales_v1(scale_h: np.ndarray, K: int) -> np.ndarray:
    M = scale_h.shape[0]
    PM = padded_m(M)
    full = np.ones(PM, np.float16)
    full[:M] = scale_h
    idx = np_ascale_v1_indices(PM, K)
    out = np.empty(PM * (K // WARP_K), np.float16)
    out[idx] = full[:, None]
    return out.reshape(PM, K // WARP_K)


# --------------------------------------------------------------- synthetic

def synth_linear(M: int, K: int, N: int, seed: int = 0, outlier_frac: float = 0.01):
    """The synthetic workload the benchmark configurations describe:
    X fp16 ~ N(0,1) with 1% of channels x20, int4 weights uniform in [-7,7],
    fp16 channel scales ~ U(1e-3,1e-2), fp16 bias ~ N(0,0.02)."""
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((M, K), dtype=np.float32)
    n_out = max(1, int(np.ceil(outlier_frac * K)))
    cols = rng.permutation(K)[:n_out]
    x[:, cols] *= 20.0
    qw = rng.integers(-7, 8, size=(N, K), dtype=np.int8)
    ws = (1e-3 + 9e-3 * rng.random(N, dtype=np.float32)).astype(np.float16)
    bias = (0.02 * rng.standard_normal(N, dtype=np.float32)).astype(np.float16)
    return x.astype(np.float16), qw, ws, bias
