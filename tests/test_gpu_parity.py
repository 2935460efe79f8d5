"""GPU parity: the HIP path (through the C ABI / the Python boundary) against
the CPU oracle on identical seeded inputs.

Bars: packed int4 activations, fp16 token scales and int32 accumulators are
bit-exact; the fp16 output is compared bit-for-bit as well (every operation of
the epilogue is a correctly rounded IEEE operation on both sides), with the
stated tolerance max|err| <= 1e-3 * max|Y| as the contractual bound.
"""
import numpy as np
import pytest
import torch

import oracle as O

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def vk():
    from dsaquant_amd.kernels import vdm_w4a4

    assert vdm_w4a4.is_available(), vdm_w4a4.load_error()
    return vdm_w4a4


def t16(a):
    return torch.from_numpy(np.ascontiguousarray(a)).to(DEV)


def unpack_native(buf: np.ndarray, K: int) -> np.ndarray:
    """row-major packed int4 [R, Kp/2] -> int8 [R, K]; also checks the zero padding."""
    lo = (buf & 0xF).astype(np.int8)
    hi = (buf >> 4).astype(np.int8)
    q = np.empty((buf.shape[0], buf.shape[1] * 2), np.int8)
    q[:, 0::2], q[:, 1::2] = lo, hi
    q = np.where(q >= 8, q - 16, q).astype(np.int8)
    assert not q[:, K:].any(), "padding nibbles must be zero"
    return q[:, :K]


def pack_native(q: np.ndarray, Kp: int) -> np.ndarray:
    R, K = q.shape
    full = np.zeros((R, Kp), np.uint8)
    full[:, :K] = q.astype(np.uint8) & 0xF
    return (full[:, 0::2] | (full[:, 1::2] << 4)).astype(np.uint8)


def special_rows(x: np.ndarray) -> np.ndarray:
    x = x.copy()
    M = x.shape[0]
    if M > 12:
        x[1] = 0
        x[2, 5] = np.float16(np.nan)
        x[3, 7] = np.float16(np.inf)
        x[4, 9] = np.float16(-np.inf)
        x[5] = np.float16(6e-8)  # fp16 scale underflows to zero
        x[6] = np.float16(65504.0)
        x[7, ::2] = np.float16(-65504.0)
        x[8] = np.float16(1e-4)
        x[9, 0] = np.float16(np.nan)
        x[9, 1] = np.float16(np.inf)
        x[10] = np.float16(np.nan)
    return x


# ------------------------------------------------------------ quantizer

QUANT_SHAPES = [(257, 1536), (4096, 1536), (515, 5120), (300, 8960), (130, 13824), (100, 64), (77, 192), (33, 3072), (64, 14336),
                (19, 16384 + 64), (5, 2048)]


@pytest.mark.parametrize("M,K", QUANT_SHAPES)
@pytest.mark.parametrize("clip", [1.0, 0.95])
def test_quantizer_bit_exact(M, K, clip):
    v = vk()
    x, _, _, _ = O.synth_linear(M, K, 128, seed=M + K)
    x = special_rows(x)
    print(f"quantizer M={M} K={K} clip={clip}", flush=True)
    qn, sc = v.quantize_activation_native(t16(x), clip)
    torch.cuda.synchronize()
    want_s = O.np_row_scale(x, clip)
    got_s = sc.cpu().numpy()
    assert np.array_equal(got_s.view(np.uint16), want_s.view(np.uint16))
    want_q = O.np_quantize_rows(x, want_s)
    got_q = unpack_native(qn.cpu().numpy(), K)
    assert np.array_equal(got_q, want_q)


def test_quantizer_against_scalar_c_oracle():
    v = vk()
    x = special_rows(O.synth_linear(64, 320, 128, seed=3)[0])
    for clip in (1.0, 0.95, 0.3, 2.0):
        qn, sc = v.quantize_activation_native(t16(x), clip)
        s = O.c_row_scale(x, clip)
        assert np.array_equal(sc.cpu().numpy().view(np.uint16), s.view(np.uint16))
        assert np.array_equal(unpack_native(qn.cpu().numpy(), 320), O.c_quantize_rows(x, s))


def test_quantizer_empty_and_strided():
    v = vk()
    qn, sc = v.quantize_activation_native(torch.empty((0, 128), dtype=torch.float16, device=DEV))
    assert qn.shape == (0, v.k_padded(128) // 2) and sc.shape == (0,)
    # leading dims are flattened, bf16/fp32 inputs are cast to fp16 first (vdm_w4a4.py:182-184)
    x = torch.randn(3, 5, 256, device=DEV)
    qn, sc = v.quantize_activation_native(x)
    xh = x.half().reshape(-1, 256).cpu().numpy()
    s = O.np_row_scale(xh, 1.0)
    assert np.array_equal(sc.cpu().numpy().view(np.uint16), s.view(np.uint16))
    assert np.array_equal(unpack_native(qn.cpu().numpy(), 256), O.np_quantize_rows(xh, s))


# ------------------------------------------------------------------ GEMM

GEMM_SHAPES = [(257, 1536, 1536), (1, 128, 64), (31, 256, 192), (512, 3072, 1536), (300, 128, 8960), (1000, 1536, 5120), (256, 10240, 5120),
               (700, 384, 13824)]


@pytest.mark.parametrize("M,N,K", GEMM_SHAPES)
def test_gemm_int32_accumulators_exact(M, N, K):
    v = vk()
    rng = np.random.default_rng(M * 7 + N + K)
    qx = rng.integers(-8, 8, (M, K), dtype=np.int8)
    qw = rng.integers(-8, 8, (N, K), dtype=np.int8)
    Kp = v.k_padded(K)
    print(f"gemm acc M={M} N={N} K={K}", flush=True)
    acc = v.gemm_int32_accumulators(t16(pack_native(qx, Kp)), t16(pack_native(qw, Kp)), K)
    torch.cuda.synchronize()
    assert np.array_equal(acc.cpu().numpy(), O.np_gemm_i32(qx, qw))


def test_gemm_extreme_values_do_not_overflow():
    v = vk()
    K = 14336
    qx = np.full((64, K), -8, np.int8)
    qw = np.full((128, K), -8, np.int8)
    qw[1] = 7
    acc = v.gemm_int32_accumulators(t16(pack_native(qx, K)), t16(pack_native(qw, K)), K).cpu().numpy()
    assert (acc[:, 0] == 64 * K).all() and (acc[:, 1] == -56 * K).all()


# ----------------------------------------------------- whole linear path

LINEAR_CASES = [
    # (M, K, N, clip, bias)  -- the reference's smoke shape, config 0, skinny/ragged cases
    (257, 1536, 1536, 0.95, True),
    (4096, 1536, 4608, 1.0, True),
    (512, 1536, 3072, 1.0, True),
    (512, 5120, 10240, 1.0, False),
    (1237, 8960, 1536, 0.95, True),
    (300, 13824, 5120, 1.0, True),
    (3, 64, 128, 1.0, True),
]


@pytest.mark.parametrize("M,K,N,clip,use_bias", LINEAR_CASES)
def test_linear_matches_oracle(M, K, N, clip, use_bias):
    v = vk()
    x, qw, ws, bias = O.synth_linear(M, K, N, seed=0)
    qweight_v1 = O.np_pack_wgt_v1(qw)
    wscales_v1 = O.np_pack_wscales_v1(ws, K)
    print(f"linear M={M} K={K} N={N} clip={clip} bias={use_bias}", flush=True)
    y = v.linear_vdm_w4a4(t16(x), t16(qweight_v1), t16(wscales_v1), t16(bias) if use_bias else None, clip_ratio=clip)
    torch.cuda.synchronize()
    assert y.dtype == torch.float16 and tuple(y.shape) == (M, N)
    want, _, _, _ = O.np_linear(x, qw, ws, bias if use_bias else None, clip)
    got = y.cpu().numpy()
    err = np.abs(got.astype(np.float32) - want.astype(np.float32)).max()
    assert err <= 1e-3 * np.abs(want.astype(np.float32)).max()  # the contractual tolerance
    assert np.array_equal(got.view(np.uint16), want.view(np.uint16))  # and in fact bit-exact


def test_linear_leading_dims_bias_half_precedence_and_dtype():
    v = vk()
    x, qw, ws, bias = O.synth_linear(2 * 130, 256, 128, seed=5)
    qv1, sv1 = t16(O.np_pack_wgt_v1(qw)), t16(O.np_pack_wscales_v1(ws, 256))
    other = (bias.astype(np.float32) * 3).astype(np.float16)
    y = v.linear_vdm_w4a4(t16(x).reshape(2, 130, 256).to(torch.bfloat16), qv1, sv1, t16(other).float(), 1.0, bias_half=t16(bias))
    assert y.shape == (2, 130, 128) and y.dtype == torch.float16
    xh = torch.from_numpy(x).to(torch.bfloat16).half().numpy()  # the cast chain the wrapper applies
    want, _, _, _ = O.np_linear(xh, qw, ws, bias, 1.0)  # bias_half wins over bias
    assert np.array_equal(y.reshape(-1, 128).cpu().numpy().view(np.uint16), want.view(np.uint16))


@pytest.mark.parametrize("path", ["int8", "bf6"])
@pytest.mark.parametrize("M,K,N,use_bias", [(300, 512, 256, True), (2300, 1536, 4608, False)])
def test_bf16_output_within_tolerance(path, M, K, N, use_bias):
    """A bf16 output (not offered by the reference) on either matrix path: the fp32 product float(acc) * (as * ws), the
    fp16 bias added in fp32, one rounding to nearest even -- within half a bf16 ulp of the exact value plus the fp32
    roundings, and the same bits on both paths (the larger case runs on the tile-walking bf6 kernel and the large int8
    tiles)."""
    v = vk()
    x, qw, ws, bias = O.synth_linear(M, K, N, seed=6)
    if not use_bias:
        bias = None
    qv1, sv1 = t16(O.np_pack_wgt_v1(qw)), t16(O.np_pack_wscales_v1(ws, K))  # (a prepared weight lives with its packed tensors)
    weight = v._prepared_weight(qv1, sv1)
    old = v.matrix_path()
    got = {}
    try:
        for p in ("int8", "bf6"):
            v.set_matrix_path(p)
            got[p] = v._linear_2d(t16(x), weight, None if bias is None else t16(bias), 1.0, out_dtype=torch.bfloat16)
            assert got[p].dtype == torch.bfloat16
    finally:
        v.set_matrix_path(old)
    assert torch.equal(got["int8"].view(torch.int16), got["bf6"].view(torch.int16))
    _, _, as_h, acc = O.np_linear(x, qw, ws, bias, 1.0)
    prod = (acc.astype(np.float32) * (as_h.astype(np.float32)[:, None] * ws.astype(np.float32)[None, :])).astype(np.float32)
    if bias is not None:
        prod = (prod + bias.astype(np.float32)[None, :]).astype(np.float32)
    want = torch.from_numpy(prod).to(torch.bfloat16)  # torch rounds to nearest even
    assert torch.equal(got[path].cpu().view(torch.int16), want.view(torch.int16))
    exact = acc.astype(np.float64) * as_h.astype(np.float64)[:, None] * ws.astype(np.float64)[None, :] + (0 if bias is None else bias.astype(np.float64))
    err = np.abs(got[path].float().cpu().numpy().astype(np.float64) - exact)
    assert err.max() <= 2.0 ** -8 * np.abs(exact).max()


def test_shape_and_dtype_errors():
    v = vk()
    x = torch.zeros((4, 128), dtype=torch.float16, device=DEV)
    qw = torch.zeros((128, 64), dtype=torch.uint8, device=DEV)
    ws = torch.zeros((128, 2), dtype=torch.float16, device=DEV)
    with pytest.raises(ValueError):
        v.linear_vdm_w4a4(torch.zeros((4, 96), dtype=torch.float16, device=DEV), qw, ws)  # K % 64
    with pytest.raises(ValueError):
        v.linear_vdm_w4a4(x, qw[:64], ws[:64])  # N % 128
    with pytest.raises(ValueError):
        v.linear_vdm_w4a4(x, torch.zeros((128, 32), dtype=torch.uint8, device=DEV), ws)  # qweight [N, K/2]
    with pytest.raises(ValueError):
        v.linear_vdm_w4a4(x, qw, ws[:, :1])  # wscales [N, K/64]
    with pytest.raises(RuntimeError):
        v.linear_vdm_w4a4(x, qw.to(torch.int8), ws)  # dtype
    with pytest.raises(RuntimeError):
        v.linear_vdm_w4a4(x, qw, ws, bias=torch.zeros(64, dtype=torch.float16, device=DEV))  # bias length
    with pytest.raises(RuntimeError):
        v.linear_prequantized(torch.zeros((100, 64), dtype=torch.uint8, device=DEV), torch.zeros((100, 2), dtype=torch.float16, device=DEV), qw, ws)


# ------------------------------------------------------ v1 layout surface

def test_pack_weight_with_scale_emits_v1_layout():
    v = vk()
    rng = np.random.default_rng(7)
    N, K = 256, 320
    w = rng.standard_normal((N, K)).astype(np.float16)
    scale = (np.abs(w.astype(np.float32)).max(axis=1) / 7).astype(np.float16)
    qweight, packed_scales, channel_scales = v.pack_weight_with_scale(t16(w), t16(scale))
    q = O.c_quantize_rows(w, scale)
    assert np.array_equal(qweight.cpu().numpy(), O.c_pack_wgt_v1(q))
    assert np.array_equal(packed_scales.cpu().numpy().view(np.uint16), O.c_pack_wscales_v1(scale, K).view(np.uint16))
    assert np.array_equal(channel_scales.cpu().numpy().view(np.uint16), scale.view(np.uint16))
    # derived scales: absmax / 7 with clip 1 (vdm_w4a4_kernel.cu:730-763)
    q2, p2, s2 = v.quantize_weight_per_channel(t16(w))
    s_want = O.c_row_scale(w, 1.0)
    assert np.array_equal(s2.cpu().numpy().view(np.uint16), s_want.view(np.uint16))
    assert np.array_equal(q2.cpu().numpy(), O.c_pack_wgt_v1(O.c_quantize_rows(w, s_want)))
    assert np.array_equal(p2.cpu().numpy().view(np.uint16), O.c_pack_wscales_v1(s_want, K).view(np.uint16))


def test_weight_relayout_roundtrip_and_cache():
    from dsaquant_amd import _lib

    v = vk()
    lib = _lib.load()
    rng = np.random.default_rng(8)
    N, K = 384, 448
    qw = rng.integers(-8, 8, (N, K), dtype=np.int8)
    v1 = t16(O.np_pack_wgt_v1(qw))
    ws = rng.random(N).astype(np.float16)
    sv1 = t16(O.np_pack_wscales_v1(ws, K))
    native, plain = v._native_weights(v1, sv1)
    assert v._native_weights(v1, sv1)[0] is native  # cached
    assert np.array_equal(unpack_native(native.cpu().numpy(), K), qw)
    assert np.array_equal(plain.cpu().numpy().view(np.uint16), ws.view(np.uint16))
    back = torch.empty_like(v1)
    _lib.check(lib.vdmq_weight_native_to_v1(native.data_ptr(), back.data_ptr(), N, K, None))
    torch.cuda.synchronize()
    assert torch.equal(back, v1)


def test_quantize_activation_per_token_v1_and_prequantized():
    v = vk()
    M, K, N = 300, 192, 256
    x, qw, ws, _ = O.synth_linear(M, K, N, seed=9)
    qact, ascales, act_scales = v.quantize_activation_per_token(t16(x), 0.95)
    s = O.c_row_scale(x, 0.95)
    q = O.c_quantize_rows(x, s)
    assert qact.shape == (512, K // 2) and ascales.shape == (512, K // 64) and act_scales.shape == (M,)
    assert np.array_equal(qact.cpu().numpy(), O.c_pack_act_v1(q))
    assert np.array_equal(ascales.cpu().numpy().view(np.uint16), O.c_pack_ascales_v1(s, K).view(np.uint16))
    assert np.array_equal(act_scales.cpu().numpy().view(np.uint16), s.view(np.uint16))
    y = v.linear_prequantized(qact, ascales, t16(O.np_pack_wgt_v1(qw)), t16(O.np_pack_wscales_v1(ws, K)))
    assert y.shape == (512, N)
    want = O.np_epilogue(O.np_gemm_i32(q, qw), s, ws, None)
    got = y.cpu().numpy()
    assert np.array_equal(got[:M].view(np.uint16), want.view(np.uint16))
    assert not got[M:].any()  # padded rows: zero activations, scale 1


def test_prepared_weights_one_form_per_layer_made_from_the_v1_buffers():
    """A packed weight is relaid straight from its v1 buffers into the form its calls use and only that form is kept:
    bf6 blocks made ahead are dropped when the calls turn out to take the int8 path (and the other way round), a
    non-contiguous qweight is not relaid per call, tensors made under inference_mode (no version counter) work, an
    in-place write to the packed buffer is noticed, and the direct v1 -> bf6 relayout writes the bytes of the two-step one."""
    from dsaquant_amd import _lib

    v = vk()
    lib = _lib.load()
    M, K, N = 300, 448, 384
    x, qw, ws, bias = O.synth_linear(M, K, N, seed=12)
    want = O.np_linear(x, qw, ws, bias, 1.0)[0]
    qv1, sv1 = t16(O.np_pack_wgt_v1(qw)), t16(O.np_pack_wscales_v1(ws, K))
    pw = v.prepare_weight(qv1, sv1, path="bf6")  # made ahead for calls on the bf6 path
    assert pw.bf6 is not None and pw.native is None
    native = torch.empty((N, v.k_padded(K) // 2), dtype=torch.uint8, device=DEV)
    two_step = torch.empty_like(pw.bf6)
    _lib.check(lib.vdmq_weight_v1_to_native(qv1.data_ptr(), native.data_ptr(), N, K, None))
    _lib.check(lib.vdmq_native_to_bf6(native.data_ptr(), N, K, two_step.data_ptr(), None))
    assert torch.equal(pw.bf6, two_step)
    y = v.linear_vdm_w4a4(t16(x), qv1, sv1, t16(bias))  # 300 rows: the int8 path under "auto"
    assert np.array_equal(y.cpu().numpy().view(np.uint16), want.view(np.uint16))
    assert v._prepared_weight(qv1, sv1) is pw and pw.native is not None and pw.bf6 is None
    assert pw.extra_bytes() == N * v.k_padded(K) // 2 + 2 * N
    old = v.matrix_path()
    v.set_matrix_path("bf6")
    try:
        y = v.linear_vdm_w4a4(t16(x), qv1, sv1, t16(bias))
        assert np.array_equal(y.cpu().numpy().view(np.uint16), want.view(np.uint16))
        assert pw.native is not None and pw.bf6 is not None  # both have been used: both stay
    finally:
        v.set_matrix_path(old)
    # non-contiguous packed buffers (a strided view): one contiguous copy and one relayout, kept with the view
    wide = torch.zeros((N, K), dtype=torch.uint8, device=DEV)
    wide[:, : K // 2] = qv1
    view = wide[:, : K // 2]
    assert not view.is_contiguous()
    y1 = v.linear_vdm_w4a4(t16(x), view, sv1, t16(bias))
    first = v._prepared_weight(view, sv1)
    y2 = v.linear_vdm_w4a4(t16(x), view, sv1, t16(bias))
    assert v._prepared_weight(view, sv1) is first and torch.equal(y1, y2)
    assert np.array_equal(y1.cpu().numpy().view(np.uint16), want.view(np.uint16))
    # an in-place write is a new weight
    qw2 = qw.copy()
    qw2[0] = -qw2[0].clip(-7, 7)
    qv1.copy_(t16(O.np_pack_wgt_v1(qw2)))
    y = v.linear_vdm_w4a4(t16(x), qv1, sv1, t16(bias))
    assert v._prepared_weight(qv1, sv1) is not pw
    assert np.array_equal(y.cpu().numpy().view(np.uint16), O.np_linear(x, qw2, ws, bias, 1.0)[0].view(np.uint16))
    # tensors created under inference_mode keep no version counter
    with torch.inference_mode():
        qi, si = t16(O.np_pack_wgt_v1(qw)), t16(O.np_pack_wscales_v1(ws, K))
        assert qi.is_inference()
        for _ in range(2):
            y = v.linear_vdm_w4a4(t16(x), qi, si, t16(bias))
        q3, k3, v3 = v.linear_vdm_w4a4_qkv(t16(x), qi, si, qi, si, qi, si, t16(bias), None, None)
        assert torch.equal(q3, y) and torch.equal(k3, v3)
    assert np.array_equal(y.cpu().numpy().view(np.uint16), want.view(np.uint16))


# --------------------------------------------------------------- fused QKV

def test_fused_qkv_is_bitwise_three_separate_calls():
    """What the reference's tests/test_vdm_qkv_fuse_smoke.py compares."""
    v = vk()
    M, K, N = 257, 1536, 1536
    x = O.synth_linear(M, K, N, seed=2)[0]
    parts = [O.synth_linear(8, K, N, seed=20 + i) for i in range(3)]
    W = [t16(O.np_pack_wgt_v1(p[1])) for p in parts]
    S = [t16(O.np_pack_wscales_v1(p[2], K)) for p in parts]
    B = [t16(p[3]) for p in parts]
    xt = t16(x).reshape(1, M, K)
    sep = [v.linear_vdm_w4a4(xt, W[i], S[i], B[i], clip_ratio=0.95) for i in range(3)]
    q, k, val = v.linear_vdm_w4a4_qkv(xt, W[0], S[0], W[1], S[1], W[2], S[2], B[0], None, B[2], clip_ratio=0.95)
    assert q.shape == (1, M, N) and q.data_ptr() != k.data_ptr()
    assert torch.equal(q, sep[0]) and torch.equal(val, sep[2])
    k_nobias = v.linear_vdm_w4a4(xt, W[1], S[1], None, clip_ratio=0.95)
    assert torch.equal(k, k_nobias)  # a missing bias is a zero bias: h + 0 == h in fp16
    # cached concatenation path
    wq = torch.cat(W, 0).contiguous()
    sq = torch.cat(S, 0).contiguous()
    bq = torch.cat(B, 0).contiguous()
    q2, k2, v2 = v.linear_vdm_w4a4_qkv(xt, W[0], S[0], W[1], S[1], W[2], S[2], clip_ratio=0.95, w_qkv_packed=wq, w_qkv_scale=sq, qkv_bias_half=bq)
    assert torch.equal(q2, sep[0]) and torch.equal(k2, sep[1]) and torch.equal(v2, sep[2])


@pytest.mark.parametrize("M,K,n", [(1000, 1536, 1536), (8200, 512, 1536), (3000, 256, 128)])
def test_split_outputs_are_the_bits_of_the_strided_views(each_matrix_path, M, K, n):
    """Fused QKV with q, k, v written as three contiguous tensors by the GEMM epilogue, and head-major
    ([3 * heads, M, 128]): the same bits as splitting the one [M, 3n] result (vdm_w4a4.py:297-298, attention.py:165-172
    of the reference); raw C-ABI call with a part stride larger than a part; the Python entries; bad splits refused."""
    from dsaquant_amd import _lib, fused_ops

    v = vk()
    lib = _lib.load()
    x = O.synth_linear(M, K, 128, seed=n)[0]
    parts = [O.synth_linear(1, K, n, seed=50 + i) for i in range(3)]
    W = [t16(O.np_pack_wgt_v1(p[1])) for p in parts]
    S = [t16(O.np_pack_wscales_v1(p[2], K)) for p in parts]
    B = [t16(p[3]) for p in parts]
    xt = t16(x)
    print(f"split outputs M={M} K={K} n={n} path={each_matrix_path}", flush=True)
    q0, k0, v0 = v.linear_vdm_w4a4_qkv(xt, W[0], S[0], W[1], S[1], W[2], S[2], B[0], B[1], B[2], clip_ratio=0.95)
    assert not q0.is_contiguous()
    q1, k1, v1 = v.linear_vdm_w4a4_qkv(xt, W[0], S[0], W[1], S[1], W[2], S[2], B[0], B[1], B[2], clip_ratio=0.95, contiguous_outputs=True)
    assert all(t.is_contiguous() and t.shape == (M, n) for t in (q1, k1, v1))
    assert torch.equal(q1, q0) and torch.equal(k1, k0) and torch.equal(v1, v0)
    want = O.np_linear(x[:64], parts[1][1], parts[1][2], parts[1][3], 0.95)[0]
    assert np.array_equal(k1[:64].cpu().numpy().view(np.uint16), want.view(np.uint16))
    # head-major through the prepared-weight entry: [3 * heads, M, 128]
    weight = v._prepared([(W[i], S[i]) for i in range(3)])
    heads = v.linear_vdm_w4a4_prepared(xt, weight, torch.cat(B), 0.95, split_cols=128)
    assert heads.shape == (3 * n // 128, M, 128) and heads.is_contiguous()
    assert torch.equal(heads.permute(1, 0, 2).reshape(M, 3 * n), torch.cat([q0, k0, v0], dim=1))
    # LayerNorm input + split, against LayerNorm input without
    rng = np.random.default_rng(1)
    a, b = t16((0.2 * rng.standard_normal((1, K))).astype(np.float16)), t16((0.3 * rng.standard_normal((1, K))).astype(np.float16))
    whole = fused_ops.linear_fused(fused_ops.LnInput(xt, a, b, 1e-6), weight, None, None, 0.95, bias_half=torch.cat(B))
    three = fused_ops.linear_fused(fused_ops.LnInput(xt, a, b, 1e-6), weight, None, None, 0.95, bias_half=torch.cat(B), split_cols=n)
    assert torch.equal(three.permute(1, 0, 2).reshape(M, 3 * n), whole)
    # raw C ABI on the int8 path: parts one row further apart than they are long, the gap untouched
    qn, sc = v.quantize_activation_native(xt, 0.95)
    out = torch.full((3, M + 1, n), -3.0, dtype=torch.float16, device=DEV)
    _lib.check(lib.vdmq_gemm_w4a4_split(qn.data_ptr(), sc.data_ptr(), weight.operand(False).data_ptr(), weight.wscale.data_ptr(),
                                        torch.cat(B).data_ptr(), out.data_ptr(), M, 3 * n, K, n, n, (M + 1) * n, torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()
    v.set_matrix_path("int8")
    ref = v.linear_vdm_w4a4_qkv(xt, W[0], S[0], W[1], S[1], W[2], S[2], B[0], B[1], B[2], clip_ratio=0.95)
    assert all(torch.equal(out[i, :M], ref[i]) for i in range(3)) and (out[:, M] == -3.0).all()
    fake = out.data_ptr()
    assert lib.vdmq_gemm_w4a4_split(fake, fake, fake, fake, None, fake, M, 3 * n, K, n, n + 32, M * n, None) == -2  # not a multiple of 64
    assert lib.vdmq_gemm_w4a4_split(fake, fake, fake, fake, None, fake, M, 3 * n, K, 64, n, M * n, None) == -2      # rows shorter than a part
    with pytest.raises(ValueError):
        v.linear_vdm_w4a4_prepared(xt, weight, None, 0.95, split_cols=96)


# ------------------------------------------------- GELU fused into the quantizer

def gpu_gelu_table():
    """fp16 -> fp16 GELU of the library for all 65 536 bit patterns."""
    from dsaquant_amd import fused_ops

    allh = np.arange(65536, dtype=np.uint16).view(np.float16)
    return allh, fused_ops.gelu_tanh(t16(allh)).cpu().numpy()


def test_gelu_table_within_one_ulp_of_the_correctly_rounded_value():
    """Floating-point part of the fused path, tolerance stated here: for every fp16 input the library's GELU is
    within 1 fp16 ulp of the correctly rounded float64 value (and equal to it for more than 99.5 % of them);
    NaN exactly where the formula gives NaN (NaN inputs and -inf)."""
    allh, got = gpu_gelu_table()
    want = O.np_gelu_tanh_f16(allh)
    assert np.array_equal(np.isnan(got), np.isnan(want))
    ok = ~np.isnan(want)
    assert np.array_equal(np.isinf(got[ok]), np.isinf(want[ok]))
    fin = ok & ~np.isinf(want)
    # ordered-integer distance; +0 and -0 count as equal
    def key(h):
        b = h.view(np.int16).astype(np.int32)
        return np.where(b < 0, -(b & 0x7FFF), b)
    ulp = np.abs(key(got[fin]) - key(want[fin]))
    print("gelu table: max ulp", ulp.max(), "inexact", int((ulp != 0).sum()), flush=True)
    assert ulp.max() <= 1
    assert (ulp != 0).mean() < 0.005


@pytest.mark.parametrize("M,K", [(515, 5120), (130, 13824), (257, 1536), (19, 16384 + 64)])
def test_fused_gelu_quantizer_is_the_quantizer_of_the_gelu_values(M, K):
    """Integer part, bit-exact: quantize(act='gelu_tanh')(x) == oracle quantizer applied to the library's own fp16
    GELU values of x (looked up in its 65 536-entry table), scales included."""
    v = vk()
    _, table = gpu_gelu_table()
    x = special_rows((3.0 * O.synth_linear(M, K, 128, seed=M + K)[0].astype(np.float32)).astype(np.float16))
    print(f"fused gelu quantizer M={M} K={K}", flush=True)
    for clip in (1.0, 0.95):
        qn, sc = v.quantize_activation_native(t16(x), clip, act="gelu_tanh")
        torch.cuda.synchronize()
        g = table[x.view(np.uint16)]
        want_s = O.np_row_scale(g, clip)
        assert np.array_equal(sc.cpu().numpy().view(np.uint16), want_s.view(np.uint16))
        assert np.array_equal(unpack_native(qn.cpu().numpy(), K), O.np_quantize_rows(g, want_s))


def test_linear_gelu_equals_unfused_chain_and_oracle():
    from dsaquant_amd import fused_ops

    v = vk()
    M, K, N = 1237, 8960, 1536
    x, qw, ws, bias = O.synth_linear(M, K, N, seed=4)
    x = (2.0 * x.astype(np.float32)).astype(np.float16)
    qv1, sv1, b = t16(O.np_pack_wgt_v1(qw)), t16(O.np_pack_wscales_v1(ws, K)), t16(bias)
    y = fused_ops.linear_gelu_vdm_w4a4(t16(x).reshape(1, M, K), qv1, sv1, b, clip_ratio=1.0)
    assert tuple(y.shape) == (1, M, N) and y.dtype == torch.float16
    y2 = v.linear_vdm_w4a4(fused_ops.gelu_tanh(t16(x)), qv1, sv1, b, clip_ratio=1.0)  # three kernels
    assert torch.equal(y[0], y2)
    _, table = gpu_gelu_table()
    want = O.np_linear(table[x.view(np.uint16)], qw, ws, bias, 1.0)[0]
    assert np.array_equal(y[0].cpu().numpy().view(np.uint16), want.view(np.uint16))
    with pytest.raises(ValueError):
        v.quantize_activation_native(t16(x), 1.0, act="relu")


# ---------------------------------- LayerNorm + modulation fused into the quantizer

def spacing16(v):
    """fp16 ulp at magnitude v (subnormal spacing below 2^-14)."""
    v = np.maximum(np.abs(v.astype(np.float64)), 2.0 ** -14)
    return 2.0 ** (np.floor(np.log2(v)) - 10)


LN_CASES = [
    # (B, L, K, per_token)
    (2, 300, 1536, False), (1, 515, 5120, False), (3, 77, 3072, True), (1, 33, 64, False), (1, 19, 16384, False), (2, 64, 8960, True)]


@pytest.mark.parametrize("B,L,K,per_token", LN_CASES)
@pytest.mark.parametrize("mode", ["modulate", "affine"])
def test_fused_layer_norm_quantizer(B, L, K, per_token, mode):
    """Floating-point part (tolerance stated here): the library's fp32 LayerNorm may land one fp16 ulp from the
    oracle's (float64 statistics); carried through the reference's fp16 chain ln * (1 + scale) + shift that bounds
    |h - oracle| by ulp(ln) * |1 + scale| + ulp(product) + ulp(h); in affine mode (fp32, one rounding) by 1 ulp(h) plus
    2^-21 of the two terms' magnitudes (fp32 rounding where they cancel).  On more
    than 99 % of the elements the two are equal.  Integer part, bit-exact:
    the fused quantizer's output is the oracle quantizer's on the library's own h; the fused linear equals the
    three-kernel chain."""
    from dsaquant_amd import fused_ops

    v = vk()
    rng = np.random.default_rng(B * 1000 + L + K)
    eps = 1e-6
    x = (rng.standard_normal((B, L, K)) * 2.0 + 0.25).astype(np.float32)
    x[..., rng.integers(0, K, max(1, K // 100))] *= 15.0
    x = x.astype(np.float16)
    nv = (B, L, K) if per_token else (B, 1, K)
    a = (0.2 * rng.standard_normal(nv)).astype(np.float16)
    b = (0.3 * rng.standard_normal(nv)).astype(np.float16)
    if mode == "affine":
        a = (1.0 + a.astype(np.float32)).astype(np.float16)
    print(f"fused LN {mode} B={B} L={L} K={K} per_token={per_token}", flush=True)
    pre = fused_ops.LnInput(t16(x), t16(a), t16(b), eps, mode)
    h_gpu = pre.materialize().cpu().numpy()
    rpv = 1 if per_token else L
    x2 = x.reshape(-1, K)
    if mode == "modulate":
        want, aux = O.np_ln_modulate_f16(x2, a.reshape(-1, K), b.reshape(-1, K), eps, rpv)
        tol = spacing16(aux["ln"]) * np.abs(aux["s1"].astype(np.float64)) + spacing16(aux["p"]) + spacing16(want)
    else:
        want = O.np_ln_affine_f16(x2, a.reshape(-1, K), b.reshape(-1, K), eps, rpv)
        # one rounding to fp16, plus the fp32 rounding of the two terms where they cancel
        terms = np.abs(O.np_layer_norm_f64(x2, eps) * np.repeat(a.reshape(-1, K), rpv, axis=0)) + np.abs(np.repeat(b.reshape(-1, K), rpv, axis=0))
        tol = spacing16(want) + 2.0 ** -21 * terms
    got = h_gpu.reshape(-1, K)
    err = np.abs(got.astype(np.float64) - want.astype(np.float64))
    assert (err <= tol).all(), float((err / tol).max())
    assert (got.view(np.uint16) != want.view(np.uint16)).mean() < 0.01
    for clip in (1.0, 0.95):
        qn, sc = pre.quantize(clip)
        want_s = O.np_row_scale(got, clip)
        assert np.array_equal(sc.cpu().numpy().view(np.uint16), want_s.view(np.uint16))
        assert np.array_equal(unpack_native(qn.cpu().numpy(), K), O.np_quantize_rows(got, want_s))
    if K <= 5120:
        N = 256
        _, qw, ws, bias = O.synth_linear(1, K, N, seed=K)
        qv1, sv1, bb = t16(O.np_pack_wgt_v1(qw)), t16(O.np_pack_wscales_v1(ws, K)), t16(bias)
        y = fused_ops.linear_ln_vdm_w4a4(pre, qv1, sv1, bb, clip_ratio=0.95)
        y3 = v.linear_vdm_w4a4(pre.materialize(), qv1, sv1, bb, clip_ratio=0.95)
        assert tuple(y.shape) == (B, L, N) and torch.equal(y, y3)


def test_fused_layer_norm_argument_errors():
    from dsaquant_amd import fused_ops

    x = torch.randn(2, 10, 128, device=DEV).half()
    with pytest.raises(ValueError):
        fused_ops.LnInput(x, torch.zeros(3, 128, device=DEV), torch.zeros(3, 128, device=DEV), 1e-6)  # 3 does not divide 20
    with pytest.raises(ValueError):
        fused_ops.LnInput(x, torch.zeros(2, 128, device=DEV), torch.zeros(1, 128, device=DEV), 1e-6)
    with pytest.raises(ValueError):
        fused_ops.LnInput(x, torch.zeros(2, 128, device=DEV), torch.zeros(2, 128, device=DEV), 1e-6, mode="rms")
    big = torch.randn(4, 16384 + 64, device=DEV).half()
    pre = fused_ops.LnInput(big, torch.zeros(1, 16384 + 64, device=DEV), torch.zeros(1, 16384 + 64, device=DEV), 1e-6)
    with pytest.raises(RuntimeError):
        pre.quantize()


# ------------------------------------- gated residual update in the GEMM epilogue

@pytest.mark.parametrize("B,L,K,N,gate_kind", [
    (2, 150, 1536, 1536, "batch"),      # 128 x 128 tiles
    (1, 8197, 1536, 4224, "batch"),     # 256 x 128 tiles
    (1, 8197, 2048, 8448, "token"),     # 256 x 256 tiles, one gate vector per token
    (3, 100, 320, 256, "none"),         # residual only (the attn2 update)
    (1, 257, 640, 384, "gate_only"),
    (8, 40, 320, 256, "batch"),         # fewer rows per gate vector than a wave owns
])
def test_gated_residual_epilogue_bit_exact(B, L, K, N, gate_kind):
    from dsaquant_amd import fused_ops

    M = B * L
    x, qw, ws, bias = O.synth_linear(M, K, N, seed=B + L)
    rng = np.random.default_rng(K + N)
    res = (2.0 * rng.standard_normal((B, L, N))).astype(np.float16)
    gate = {"batch": (B, 1, N), "token": (B, L, N), "none": None, "gate_only": (B, 1, N)}[gate_kind]
    g = None if gate is None else rng.standard_normal(gate).astype(np.float16)
    r = None if gate_kind == "gate_only" else res
    qv1, sv1, bb = t16(O.np_pack_wgt_v1(qw)), t16(O.np_pack_wscales_v1(ws, K)), t16(bias)
    print(f"gated residual B={B} L={L} K={K} N={N} gate={gate_kind}", flush=True)
    out = fused_ops.linear_fused(t16(x).reshape(B, L, K), qv1, sv1, bb, 0.95, residual=None if r is None else t16(r),
                                 gate=None if g is None else t16(g))
    torch.cuda.synchronize()
    assert tuple(out.shape) == (B, L, N)
    y = O.np_linear(x, qw, ws, bias, 0.95)[0]
    rpg = 1 if gate_kind == "token" else L
    want = O.np_gated_residual(y, None if g is None else g.reshape(-1, N), None if r is None else r.reshape(-1, N), rpg)
    assert np.array_equal(out.cpu().numpy().reshape(-1, N).view(np.uint16), want.view(np.uint16))


def test_gated_residual_in_place_through_the_c_abi_and_errors():
    """out == residual (the in-place hidden-state update) through vdmq_gemm_w4a4_ex; argument errors."""
    from dsaquant_amd import _lib, fused_ops

    v = vk()
    lib = _lib.load()
    M, K, N = 700, 512, 640
    x, qw, ws, bias = O.synth_linear(M, K, N, seed=9)
    rng = np.random.default_rng(2)
    res = rng.standard_normal((M, N)).astype(np.float16)
    g = rng.standard_normal((1, N)).astype(np.float16)
    qn, sc = v.quantize_activation_native(t16(x), 1.0)
    wn, wsd, bd, gd = t16(pack_native(qw, v.k_padded(K))), t16(ws), t16(bias), t16(g)
    hidden = t16(res).clone()
    s = torch.cuda.current_stream().cuda_stream
    _lib.check(lib.vdmq_gemm_w4a4_ex(qn.data_ptr(), sc.data_ptr(), wn.data_ptr(), wsd.data_ptr(), bd.data_ptr(), gd.data_ptr(), N, M,
                                     hidden.data_ptr(), N, hidden.data_ptr(), 0, M, N, K, N, s))
    torch.cuda.synchronize()
    want = O.np_gated_residual(O.np_linear(x, qw, ws, bias, 1.0)[0], g, res, M)
    assert np.array_equal(hidden.cpu().numpy().view(np.uint16), want.view(np.uint16))
    # bf16 output with a tail, bad strides
    assert lib.vdmq_gemm_w4a4_ex(qn.data_ptr(), sc.data_ptr(), wn.data_ptr(), wsd.data_ptr(), None, gd.data_ptr(), N, M, None, 0,
                                 hidden.data_ptr(), 1, M, N, K, N, s) == -1
    assert lib.vdmq_gemm_w4a4_ex(qn.data_ptr(), sc.data_ptr(), wn.data_ptr(), wsd.data_ptr(), None, gd.data_ptr(), N - 8, M, None, 0,
                                 hidden.data_ptr(), 0, M, N, K, N, s) == -2
    xt = t16(x)
    with pytest.raises(ValueError):
        fused_ops.linear_fused(xt, t16(O.np_pack_wgt_v1(qw)), t16(O.np_pack_wscales_v1(ws, K)), residual=xt)  # wrong shape
    with pytest.raises(ValueError):
        fused_ops.linear_fused(xt, t16(O.np_pack_wgt_v1(qw)), t16(O.np_pack_wscales_v1(ws, K)), gate=torch.zeros(3, N, device=DEV))


# ------------------------------------------------------------ bf6 matrix path

@pytest.fixture
def bf6_path():
    v = vk()
    old = v.matrix_path()
    v.set_matrix_path("bf6")
    yield v
    v.set_matrix_path(old)


@pytest.mark.parametrize("M,K", [(257, 1536), (100, 64), (77, 192), (515, 5120), (19, 16384 + 64)])
def test_bf6_blocks_hold_the_quantized_values(M, K):
    """native int4 -> bf6 blocks: decoding the blocks with the format's definition gives back the oracle's integers
    (layout, E3M2 codes of q / 16 and zero padding of rows to 32 and K to 128)."""
    v = vk()
    x = special_rows(O.synth_linear(M, K, 128, seed=M + K)[0])
    qn, sc = v.quantize_activation_native(t16(x), 0.95)
    blocks = v.bf6_blocks(qn, K).cpu().numpy()
    want = O.np_quantize_rows(x, O.np_row_scale(x, 0.95))
    assert np.array_equal(O.np_unpack_bf6_blocks(blocks, M, K), want.astype(np.float64))


def rows_of_blocks(blocks: torch.Tensor, M: int, K: int) -> np.ndarray:
    """Decode a bf6 operand whose rows beyond M (in the last 32-row block) are unspecified."""
    b = blocks.cpu().numpy().reshape((M + 31) // 32 * 4, -1, 384).copy()
    for r in range(M, (M + 31) // 32 * 32):  # the quantizers do not write these rows: clear them before the padding check
        b[r // 8, :, :256].reshape(-1, 2, 8, 16)[:, :, r % 8] = 0
        b[r // 8, :, 256:].reshape(-1, 2, 8, 8)[:, :, r % 8] = 0
    return O.np_unpack_bf6_blocks(b.reshape(-1), M, K)


@pytest.mark.parametrize("M,K", [(257, 1536), (100, 64), (77, 192), (515, 5120), (130, 13824), (19, 16384), (4096, 8960), (33, 3072), (2100, 13824)])
def test_bf6_quantizers_write_the_oracle_integers(M, K):
    """The quantizers that emit bf6 blocks directly (plain, GELU, LayerNorm): decoded with the format's definition,
    the blocks hold the oracle's integers (plain) / the integers of the int4 quantizer (fused producers), scales equal.
    Rows longer than 8192 make a workgroup walk several row groups once there are more groups than the chip
    holds (256 CUs x 1): (4096, 8960) gives every workgroup two, (2100, 13824) a few of them a second, ragged one."""
    from dsaquant_amd import fused_ops

    v = vk()
    x = special_rows((2.0 * O.synth_linear(M, K, 128, seed=M + K)[0].astype(np.float32)).astype(np.float16))
    print(f"bf6 quantizers M={M} K={K}", flush=True)
    for clip in (1.0, 0.95):
        blocks, sc = v.quantize_activation_bf6(t16(x), clip)
        want_s = O.np_row_scale(x, clip)
        assert np.array_equal(sc.cpu().numpy().view(np.uint16), want_s.view(np.uint16))
        assert np.array_equal(rows_of_blocks(blocks, M, K), O.np_quantize_rows(x, want_s).astype(np.float64))
    blocks, sc = v.quantize_activation_bf6(t16(x), 1.0, act="gelu_tanh")
    qn, sc4 = v.quantize_activation_native(t16(x), 1.0, act="gelu_tanh")
    assert torch.equal(sc.view(torch.int16), sc4.view(torch.int16))
    assert np.array_equal(rows_of_blocks(blocks, M, K), unpack_native(qn.cpu().numpy(), K).astype(np.float64))
    rng = np.random.default_rng(M)
    a, b = (0.2 * rng.standard_normal((1, K))).astype(np.float16), (0.3 * rng.standard_normal((1, K))).astype(np.float16)
    xf = np.where(np.isfinite(x), x, np.float16(1.0))
    for mode in ("modulate", "affine"):
        pre = fused_ops.LnInput(t16(xf), t16(a), t16(b), 1e-6, mode)
        blocks, sc = pre.quantize(0.95, bf6=True)
        qn, sc4 = pre.quantize(0.95)
        assert torch.equal(sc.view(torch.int16), sc4.view(torch.int16))
        assert np.array_equal(rows_of_blocks(blocks, M, K), unpack_native(qn.cpu().numpy(), K).astype(np.float64))


@pytest.mark.parametrize("M,N,K", [(257, 1536, 1536), (1, 128, 64), (300, 128, 8960), (700, 384, 13824), (4100, 8320, 640), (8200, 8320, 2304)])
def test_bf6_accumulators_exact(M, N, K):
    v = vk()
    rng = np.random.default_rng(M * 7 + N + K)
    qx = rng.integers(-8, 8, (M, K), dtype=np.int8)
    qw = rng.integers(-8, 8, (N, K), dtype=np.int8)
    Kp = v.k_padded(K)
    print(f"bf6 acc M={M} N={N} K={K}", flush=True)
    acc = v.gemm_int32_accumulators(t16(pack_native(qx, Kp)), t16(pack_native(qw, Kp)), K, path="bf6")
    torch.cuda.synchronize()
    assert np.array_equal(acc.cpu().numpy(), O.np_gemm_i32(qx, qw))


def test_both_matrix_paths_agree_on_random_shapes():
    """Thirty seeded shapes (ragged M, every multiple of 128 / 64 allowed for N / K, up to several tiles and
    super-tiles) and three wide ones that take the bf6 kernel's contiguous tile order with ragged edges: the
    accumulators of the two matrix paths are the same integers, and the first shapes are also checked against the
    integer product on the CPU."""
    v = vk()
    rng = np.random.default_rng(2024)
    wide = [(260, 12544, 2048), (1100, 13824, 4096), (2300, 12288, 2112)]  # >= 48 tile columns, K >= 2048: contiguous runs
    for i in range(30 + len(wide)):
        if i >= 30:
            M, N, K = wide[i - 30]
        else:
            M = int(rng.integers(1, 2600))
            N = 128 * int(rng.integers(1, 20))
            K = 64 * int(rng.integers(1, 70))
        qx = rng.integers(-8, 8, (M, K), dtype=np.int8)
        qw = rng.integers(-8, 8, (N, K), dtype=np.int8)
        Kp = v.k_padded(K)
        print(f"paths agree M={M} N={N} K={K}", flush=True)
        xn, wn = t16(pack_native(qx, Kp)), t16(pack_native(qw, Kp))
        a8 = v.gemm_int32_accumulators(xn, wn, K, path="int8")
        a6 = v.gemm_int32_accumulators(xn, wn, K, path="bf6")
        assert torch.equal(a8, a6), (M, N, K)
        if i < 6:
            assert np.array_equal(a6.cpu().numpy(), O.np_gemm_i32(qx, qw))


def test_matrix_paths_give_the_same_fp16_outputs():
    """Twenty seeded problems through the whole linear (quantizer, GEMM, epilogue) on either matrix path: the fp16
    outputs are the same bits, with and without bias, plain and with the gated residual tail.  The shapes cover what
    the bf6 launcher chooses between: several rounds of tiles per CU (the kernel that walks tiles), few tiles, long
    K, wide N, ragged M throughout."""
    from dsaquant_amd import fused_ops

    v = vk()
    rng = np.random.default_rng(77)
    old = v.matrix_path()
    try:
        for i in range(20):
            kind = i % 4
            if kind == 0:
                M, N, K = int(rng.integers(3000, 12000)), 128 * int(rng.integers(8, 36)), 64 * int(rng.integers(1, 16))
            elif kind == 1:
                M, N, K = int(rng.integers(1, 3000)), 128 * int(rng.integers(1, 16)), 64 * int(rng.integers(40, 225))
            elif kind == 2:
                M, N, K = int(rng.integers(1, 700)), 128 * int(rng.integers(1, 12)), 64 * int(rng.integers(1, 40))
            else:
                M, N, K = int(rng.integers(200, 3000)), 128 * int(rng.integers(60, 120)), 64 * int(rng.integers(8, 40))
            x, qw, ws, bias = O.synth_linear(M, K, N, seed=i)
            tail = i % 3
            print(f"same fp16 outputs M={M} N={N} K={K} tail={tail}", flush=True)
            args = (t16(x), t16(O.np_pack_wgt_v1(qw)), t16(O.np_pack_wscales_v1(ws, K)), t16(bias) if i % 2 else None)
            res = t16(rng.standard_normal((M, N)).astype(np.float16)) if tail else None
            gate = t16(rng.standard_normal((1, N)).astype(np.float16)) if tail == 2 else None
            got = {}
            for path in ("int8", "bf6"):
                v.set_matrix_path(path)
                got[path] = (fused_ops.linear_fused(*args, clip_ratio=0.95, residual=res, gate=gate) if tail
                             else v.linear_vdm_w4a4(*args, clip_ratio=0.95))
            torch.cuda.synchronize()
            assert torch.equal(got["int8"].view(torch.int16), got["bf6"].view(torch.int16)), (M, N, K, tail)
    finally:
        v.set_matrix_path(old)


def test_bf6_extreme_values_stay_exact():
    """|acc| up to 64 * K = 2^20 * 0.875 with K = 14336: exact in the fp32 accumulator."""
    v = vk()
    K = 14336
    qx = np.full((64, K), -8, np.int8)
    qw = np.full((128, K), -8, np.int8)
    qw[1] = 7
    acc = v.gemm_int32_accumulators(t16(pack_native(qx, K)), t16(pack_native(qw, K)), K, path="bf6").cpu().numpy()
    assert (acc[:, 0] == 64 * K).all() and (acc[:, 1] == -56 * K).all()


@pytest.mark.parametrize("M,K,N,clip,use_bias", LINEAR_CASES)
def test_bf6_linear_matches_oracle(bf6_path, M, K, N, clip, use_bias):
    v = bf6_path
    x, qw, ws, bias = O.synth_linear(M, K, N, seed=0)
    print(f"bf6 linear M={M} K={K} N={N}", flush=True)
    y = v.linear_vdm_w4a4(t16(x), t16(O.np_pack_wgt_v1(qw)), t16(O.np_pack_wscales_v1(ws, K)), t16(bias) if use_bias else None, clip_ratio=clip)
    torch.cuda.synchronize()
    want = O.np_linear(x, qw, ws, bias if use_bias else None, clip)[0]
    assert np.array_equal(y.cpu().numpy().view(np.uint16), want.view(np.uint16))


def test_bf6_linear_through_the_c_abi():
    """vdmq_linear_w4a4_bf6 with an input row stride, GELU fused, against the oracle chain; short workspace refused."""
    from dsaquant_amd import _lib

    v = vk()
    lib = _lib.load()
    M, K, N, ldx = 300, 320, 256, 384
    x, qw, ws, bias = O.synth_linear(M, K, N, seed=31)
    xs = torch.full((M, ldx), 1000.0, dtype=torch.float16, device=DEV)
    xs[:, :K] = t16(x)
    wb = v.bf6_blocks(t16(pack_native(qw, v.k_padded(K))), K)
    wsd, bd = t16(ws), t16(bias)
    out = torch.empty((M, N), dtype=torch.float16, device=DEV)
    need = int(lib.vdmq_workspace_bytes_bf6(M, K))
    wsp = torch.empty(need, dtype=torch.uint8, device=DEV)
    s = torch.cuda.current_stream().cuda_stream
    _lib.check(lib.vdmq_linear_w4a4_bf6(xs.data_ptr(), M, K, ldx, 1.0, _lib.VDMQ_ACT_GELU_TANH, wb.data_ptr(), wsd.data_ptr(), bd.data_ptr(),
                                        out.data_ptr(), _lib.VDMQ_OUT_F16, N, N, wsp.data_ptr(), need, s))
    torch.cuda.synchronize()
    _, table = gpu_gelu_table()
    want = O.np_linear(table[x.view(np.uint16)], qw, ws, bias, 1.0)[0]
    assert np.array_equal(out.cpu().numpy().view(np.uint16), want.view(np.uint16))
    assert lib.vdmq_linear_w4a4_bf6(xs.data_ptr(), M, K, ldx, 1.0, 0, wb.data_ptr(), wsd.data_ptr(), bd.data_ptr(), out.data_ptr(), 0, N, N,
                                    wsp.data_ptr(), need - 1, s) == -4


def test_bf6_fused_paths_equal_the_int8_ones(bf6_path):
    """LayerNorm input, GELU input and gated residual through the bf6 GEMM: bitwise equal to the int8 path."""
    from dsaquant_amd import fused_ops

    v = bf6_path
    B, L, K, N = 2, 300, 1536, 1536
    rng = np.random.default_rng(3)
    x = (rng.standard_normal((B, L, K)) * 2).astype(np.float16)
    a, b = (0.2 * rng.standard_normal((B, 1, K))).astype(np.float16), (0.3 * rng.standard_normal((B, 1, K))).astype(np.float16)
    _, qw, ws, bias = O.synth_linear(1, K, N, seed=5)
    qv1, sv1, bb = t16(O.np_pack_wgt_v1(qw)), t16(O.np_pack_wscales_v1(ws, K)), t16(bias)
    res, gate = t16(rng.standard_normal((B, L, N)).astype(np.float16)), t16(rng.standard_normal((B, 1, N)).astype(np.float16))

    def run():
        pre = fused_ops.LnInput(t16(x), t16(a), t16(b), 1e-6)
        return (fused_ops.linear_fused(pre, qv1, sv1, bb, 0.95, residual=res, gate=gate),
                fused_ops.linear_fused(t16(x), qv1, sv1, bb, 1.0, act="gelu_tanh", residual=res))

    got = run()
    v.set_matrix_path("int8")
    want = run()
    assert torch.equal(got[0], want[0]) and torch.equal(got[1], want[1])


# --------------------------- large-tile configuration, strided C-ABI calls

@pytest.mark.parametrize("M,N,K", [(4100, 8320, 640), (8200, 8320, 2304)])
def test_mid_and_large_tile_configurations_accumulators(M, N, K):
    """The library picks the tile configuration from the shape: 128 x 128 tiles for the small shapes above,
    256 x 128 for a few hundred large tiles or short K (first case), 256 x 256 beyond (second case).
    Both are ragged in M and N; the first also in K."""
    v = vk()
    rng = np.random.default_rng(5)
    qx = rng.integers(-8, 8, (M, K), dtype=np.int8)
    qw = rng.integers(-8, 8, (N, K), dtype=np.int8)
    Kp = v.k_padded(K)
    print(f"tile-config acc M={M} N={N} K={K}", flush=True)
    acc = v.gemm_int32_accumulators(t16(pack_native(qx, Kp)), t16(pack_native(qw, Kp)), K)
    torch.cuda.synchronize()
    assert np.array_equal(acc.cpu().numpy(), O.np_gemm_i32(qx, qw))


@pytest.mark.parametrize("M,K,N", [(8197, 1536, 4224), (8197, 2048, 8448)])
def test_mid_and_large_tile_configurations_linear(M, K, N):
    v = vk()
    x, qw, ws, bias = O.synth_linear(M, K, N, seed=11)
    x = special_rows(x)
    print(f"tile-config linear M={M} K={K} N={N}", flush=True)
    y = v.linear_vdm_w4a4(t16(x), t16(O.np_pack_wgt_v1(qw)), t16(O.np_pack_wscales_v1(ws, K)), t16(bias), clip_ratio=0.95)
    torch.cuda.synchronize()
    want = O.np_linear(x, qw, ws, bias, 0.95)[0]
    got = y.cpu().numpy()
    assert np.array_equal(got.view(np.uint16), want.view(np.uint16))


def test_c_abi_with_row_strides():
    """vdmq_linear_w4a4 called directly with an input row stride > K and an
    output row stride > N: the columns beyond N stay untouched."""
    from dsaquant_amd import _lib

    v = vk()
    lib = _lib.load()
    M, K, N, ldx, ldo = 300, 320, 128, 384, 200
    x, qw, ws, bias = O.synth_linear(M, K, N, seed=21)
    xs = torch.full((M, ldx), 1000.0, dtype=torch.float16, device=DEV)  # the pad columns would change every row scale
    xs[:, :K] = t16(x)
    native_w = t16(pack_native(qw, v.k_padded(K)))
    out = torch.full((M, ldo), -3.0, dtype=torch.float16, device=DEV)
    wsb = int(lib.vdmq_workspace_bytes(M, K))
    wsp = torch.empty(wsb, dtype=torch.uint8, device=DEV)
    wsd, bd = t16(ws), t16(bias)
    print("strided C-ABI linear", flush=True)
    _lib.check(lib.vdmq_linear_w4a4(xs.data_ptr(), M, K, ldx, 1.0, native_w.data_ptr(), wsd.data_ptr(), bd.data_ptr(), out.data_ptr(), 0, N,
                                    ldo, wsp.data_ptr(), wsb, torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()
    got = out.cpu().numpy()
    want = O.np_linear(x, qw, ws, bias, 1.0)[0]
    assert np.array_equal(got[:, :N].view(np.uint16), want.view(np.uint16))
    assert (got[:, N:] == np.float16(-3.0)).all()
    # a workspace one byte short is refused before anything is launched
    assert lib.vdmq_linear_w4a4(xs.data_ptr(), M, K, ldx, 1.0, native_w.data_ptr(), wsd.data_ptr(), bd.data_ptr(), out.data_ptr(), 0, N, ldo,
                                wsp.data_ptr(), wsb - 1, torch.cuda.current_stream().cuda_stream) == -4


# ---------------------------------------------------- full-size properties

@pytest.fixture(params=["int8", "bf6"])
def each_matrix_path(request):
    v = vk()
    old = v.matrix_path()
    v.set_matrix_path(request.param)
    yield request.param
    v.set_matrix_path(old)


def test_config3_sized_rows_sampled_against_oracle_and_ragged_tail(each_matrix_path):
    """Wan-14B 720p fused QKV shape with the ragged M = 75600 + 37, on either matrix path: a sample of
    rows (including the last tile's tail) against the oracle, every row's token
    scale, and the un-ragged prefix against a second run with M = 75600."""
    v = vk()
    M, K, N = 75637, 5120, 15360
    g = torch.Generator(device="cpu").manual_seed(0)
    x = torch.randn((M, K), generator=g, dtype=torch.float32)
    cols = torch.randperm(K, generator=g)[: int(np.ceil(0.01 * K))]
    x[:, cols] *= 20
    x = x.half()
    _, qw, ws, bias = O.synth_linear(1, K, N, seed=0)
    qv1, sv1, b = t16(O.np_pack_wgt_v1(qw)), t16(O.np_pack_wscales_v1(ws, K)), t16(bias)
    xd = x.to(DEV)
    print("config-3 ragged linear", flush=True)
    y = v.linear_vdm_w4a4(xd, qv1, sv1, b, clip_ratio=1.0)
    y0 = v.linear_vdm_w4a4(xd[:75600], qv1, sv1, b, clip_ratio=1.0)
    torch.cuda.synchronize()
    assert torch.equal(y[:75600], y0)
    rows = np.concatenate([np.arange(0, 64), np.arange(37800, 37832), np.arange(75580, M)])
    want, _, _, _ = O.np_linear(x[rows].numpy(), qw, ws, bias, 1.0)
    assert np.array_equal(y[torch.from_numpy(rows).to(DEV)].cpu().numpy().view(np.uint16), want.view(np.uint16))
    # row-permutation equivariance on a shuffled block (exact)
    perm = torch.randperm(4096, generator=g)
    yp = v.linear_vdm_w4a4(xd[:4096][perm.to(DEV)], qv1, sv1, b, clip_ratio=1.0)
    assert torch.equal(yp, y[:4096][perm.to(DEV)])
    _, sc = v.quantize_activation_native(xd, 1.0)
    assert np.array_equal(sc.cpu().numpy().view(np.uint16), O.np_row_scale(x.numpy(), 1.0).view(np.uint16))


def test_config3_sized_ffn_down_long_rows(each_matrix_path):
    """Wan-14B 720p FFN-down shape (K = 13824: the quantizers' long-row forms, on the bf6 path workgroups that walk
    37 row groups each) with the ragged M = 75600 + 37: sampled rows against the oracle, every token scale against
    the scale formula evaluated by torch in fp32, prefix equality."""
    v = vk()
    M, K, N = 75637, 13824, 5120
    g = torch.Generator(device=DEV).manual_seed(11)
    xd = torch.randn((M, K), generator=g, device=DEV, dtype=torch.float16)
    xd[:, :: 97] *= 12
    _, qw, ws, bias = O.synth_linear(1, K, N, seed=2)
    qv1, sv1, b = t16(O.np_pack_wgt_v1(qw)), t16(O.np_pack_wscales_v1(ws, K)), t16(bias)
    print(f"config-3 ffn-down {each_matrix_path}", flush=True)
    y = v.linear_vdm_w4a4(xd, qv1, sv1, b, clip_ratio=0.95)
    y0 = v.linear_vdm_w4a4(xd[:75600], qv1, sv1, b, clip_ratio=0.95)
    assert torch.equal(y[:75600], y0)
    rows = torch.from_numpy(np.concatenate([np.arange(0, 40), np.arange(2040, 2060), np.arange(40000, 40024), np.arange(75590, M)])).to(DEV)
    want, _, _, _ = O.np_linear(xd[rows].cpu().numpy(), qw, ws, bias, 0.95)
    assert np.array_equal(y[rows].cpu().numpy().view(np.uint16), want.view(np.uint16))
    if each_matrix_path == "bf6":
        _, sc = v.quantize_activation_bf6(xd, 0.95)
    else:
        _, sc = v.quantize_activation_native(xd, 0.95)
    amax = xd.abs().amax(dim=1).float()
    seven = torch.full_like(amax, 7.0)  # a tensor divisor: torch turns division by a Python scalar into a multiplication
    assert torch.equal(sc.view(-1), ((amax / seven) * 0.95).half())


# ------------------------------------------------------------- HIP graphs

def test_linear_replays_from_a_hip_graph(each_matrix_path):
    """Nothing on the path allocates through HIP, synchronises or clears memory with a memset node: the whole fused
    linear (LayerNorm quantizer, GEMM with the gated residual tail) and the plain one are captured into one graph and
    replayed with new inputs, eager work and synchronisations between the replays; every replay equals the eager result."""
    from dsaquant_amd import fused_ops

    v = vk()
    B, L, K, N = 2, 1500, 1536, 1536
    rng = np.random.default_rng(9)
    _, qw, ws, bias = O.synth_linear(1, K, N, seed=4)
    qv1, sv1, b = t16(O.np_pack_wgt_v1(qw)), t16(O.np_pack_wscales_v1(ws, K)), t16(bias)

    def fresh(shape, scale=1.0):
        return t16((scale * rng.standard_normal(shape)).astype(np.float16))

    def step(x, a, sh, res, gate):
        h = fused_ops.linear_fused(fused_ops.LnInput(x, a, sh, 1e-6), qv1, sv1, b, 0.95, residual=res, gate=gate)
        return v.linear_vdm_w4a4(h, qv1, sv1, b, clip_ratio=1.0)

    statics = [fresh((B, L, K)), fresh((B, 1, K), 0.2), fresh((B, 1, K), 0.3), fresh((B, L, N)), fresh((B, 1, N))]
    step(*statics)  # first call: weight relayouts and per-device kernel attributes, outside the capture
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    print(f"graph capture {each_matrix_path}", flush=True)
    with torch.cuda.graph(graph):
        out = step(*statics)
    for it in range(3):
        new = [fresh((B, L, K), 1.0 + it), fresh((B, 1, K), 0.2), fresh((B, 1, K), 0.3), fresh((B, L, N)), fresh((B, 1, N))]
        for dst, src in zip(statics, new):
            dst.copy_(src)
        graph.replay()
        torch.cuda.synchronize()
        got = out.clone()
        want = step(*new)
        torch.cuda.synchronize()
        assert torch.equal(got, want), it


# ------------------------------------------------------- committed fixture

def test_hip_path_reproduces_the_committed_emulation_fixture():
    """Every surface of the API against tests/golden/w4a4_emulated_257x128x128.npz
    (written by the lane-level emulation of the reference's CUDA kernels)."""
    from pathlib import Path

    v = vk()
    f = np.load(Path(__file__).parent / "golden" / "w4a4_emulated_257x128x128.npz")
    x, w, wscale, bias, clip = f["x"], f["w"], f["wscale"], f["bias"], float(f["clip"])
    qweight, packed_scales, channel_scales = v.pack_weight_with_scale(t16(w), t16(wscale))
    assert np.array_equal(qweight.cpu().numpy(), f["qweight"])
    assert np.array_equal(packed_scales.cpu().numpy().view(np.uint16), f["wscales_packed"].view(np.uint16))
    qact, ascales, act_scales = v.quantize_activation_per_token(t16(x), clip)
    assert np.array_equal(qact.cpu().numpy(), f["qact"])
    assert np.array_equal(ascales.cpu().numpy().view(np.uint16), f["ascales"].view(np.uint16))
    assert np.array_equal(act_scales.cpu().numpy().view(np.uint16), f["act_scales"].view(np.uint16))
    y = v.linear_vdm_w4a4(t16(x), t16(f["qweight"]), t16(f["wscales_packed"]), t16(bias), clip_ratio=clip)
    assert np.array_equal(y.cpu().numpy().view(np.uint16), f["y"].view(np.uint16))
    native_x, _ = v.quantize_activation_native(t16(x), clip)
    native_w, _ = v._native_weights(t16(f["qweight"]), t16(f["wscales_packed"]))
    acc = v.gemm_int32_accumulators(native_x, native_w, 128)
    assert np.array_equal(acc.cpu().numpy(), f["acc"])


@pytest.mark.gpu
@pytest.mark.parametrize("tag", ["v1", "legacy"])
def test_reference_written_checkpoint_runs_through_the_kernels(tag):
    """The checkpoint the reference's own save_packed_checkpoint wrote (tests/golden/make_checkpoint_fixture.py), loaded
    with the kernel required: both QuantLinear layers give the oracle's fp16 bits for the integers and scales the
    file holds, at the module's clip ratio of 0.95 (quant_linear.py:121, :163-172)."""
    from pathlib import Path

    from dsaquant_amd.checkpoints import packed_checkpoint as pc
    from dsaquant_amd.quantization.quant_linear import QuantLinear
    from tests.toy_model import build_toy

    vk()
    golden = Path(__file__).parent / "golden"
    ckpt = pc.load_quant_checkpoint(str(golden / f"reference_written_packed_{tag}.pt"), dcp_loader=None)
    model = build_toy(QuantLinear, seed=3)
    missing, unexpected = pc.load_packed_quantized_model(model, ckpt, quant_linear_cls=QuantLinear, dtype=torch.float16,
                                                        device=torch.device("cuda:0"))
    assert missing == [] and unexpected == []
    rng = np.random.default_rng(5)
    for layer in (model.q1, model.q2):
        N, K = layer.out_features, layer.in_features
        x = rng.standard_normal((33, K)).astype(np.float16)
        x[:, 5] *= np.float16(20.0)
        x[7] = 0
        print(f"reference-written checkpoint {tag}: layer {K}->{N}", flush=True)
        y = layer(t16(x))
        torch.cuda.synchronize()
        qw = O.np_unpack_wgt_v1(layer.vdm_weight_packed.cpu().numpy(), N, K)
        ws = layer.vdm_weight_scale.cpu().numpy()
        assert np.array_equal(O.np_unpack_wscales_v1(layer.vdm_weight_scale_packed.cpu().numpy(), N, K), ws)
        bias = None if layer.bias is None else layer.bias.detach().cpu().numpy()
        want = O.np_linear(x, qw, ws, bias, 0.95)[0]
        assert y.dtype == torch.float16 and np.array_equal(y.cpu().numpy().view(np.uint16), want.view(np.uint16))
