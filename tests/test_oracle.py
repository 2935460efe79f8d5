"""Pins the CPU oracle (oracle/) before anything is compared with it.

No reference-held golden vectors exist for this path (the reference's four
test scripts draw random CUDA tensors and print error norms), so the oracle is
pinned by: exhaustive/known-answer fp16 conversions against numpy, brute-force
and closed-form special cases of the quantizer, a thread-level emulation of the
reference's CUDA packers and GEMM kernel built from the PTX ISA's fragment
tables (tests/ptx_emulation.py), textbook integer matmul, and the dense
formula the reference's own kernel smoke test prints against
(tests/test_vdm_w4a4_kernel_smoke.py:25-28 in the reference).
"""
import ctypes

import numpy as np
import pytest

import oracle as O
from tests import ptx_emulation as E


# ------------------------------------------------------------------- fp16

def test_h2f_exhaustive():
    L = O.lib()
    bits = np.arange(65536, dtype=np.uint16)
    want = bits.view(np.float16).astype(np.float32)
    got = np.array([L.vdmq_oracle_h2f(int(b)) for b in bits], np.float32)
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got[~nan].view(np.uint32), want[~nan].view(np.uint32))


def test_f2h_matches_numpy_rne():
    L = O.lib()
    rng = np.random.default_rng(1)
    vals = np.concatenate([
        rng.standard_normal(20000).astype(np.float32) * np.float32(10.0) ** rng.integers(-9, 6, 20000).astype(np.float32),
        # every fp16 value, the midpoints between neighbours, and one fp32 ulp either side of them
        np.arange(0, 0x7C00, dtype=np.uint16).view(np.float16).astype(np.float32),
        np.array([65504.0, 65519.99, 65520.0, 65536.0, 1e9, 5.96e-8, 2.98e-8, 2.9802322e-8, 2.99e-8, 1e-10, 0.0, -0.0], np.float32),
    ])
    h = np.arange(0, 0x7BFF, dtype=np.uint16).view(np.float16).astype(np.float64)
    h2 = np.arange(1, 0x7C00, dtype=np.uint16).view(np.float16).astype(np.float64)
    mid = ((h + h2) / 2).astype(np.float32)  # exact: midpoints need 12 bits
    vals = np.concatenate([vals, mid, np.nextafter(mid, np.float32(np.inf)), np.nextafter(mid, np.float32(-np.inf))])
    vals = np.concatenate([vals, -vals])
    with np.errstate(over="ignore"):
        want = vals.astype(np.float16).view(np.uint16)
    got = np.array([L.vdmq_oracle_f2h(float(v)) for v in vals], np.uint16)
    assert np.array_equal(got, want)


def test_d2h_sum_of_halves_is_single_rounding():
    L = O.lib()
    rng = np.random.default_rng(2)
    a = rng.integers(0, 0x7C00, 20000).astype(np.uint16).view(np.float16)
    b = (rng.integers(0, 0x7C00, 20000).astype(np.uint16) | (rng.integers(0, 2, 20000).astype(np.uint16) << 15)).view(np.float16)
    s = a.astype(np.float64) + b.astype(np.float64)
    with np.errstate(over="ignore"):
        want = s.astype(np.float16).view(np.uint16)  # numpy float64->float16 is correctly rounded
    got = np.array([L.vdmq_oracle_d2h(float(v)) for v in s], np.uint16)
    assert np.array_equal(got, want)


# -------------------------------------------------------------- quantizer

def _rand_x(M, K, seed, outliers=True):
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((M, K)).astype(np.float32)
    if outliers:
        x[:, rng.permutation(K)[: max(1, K // 100)]] *= 20
    return x.astype(np.float16)


@pytest.mark.parametrize("clip", [1.0, 0.95, 0.5])
def test_quantizer_c_equals_numpy(clip):
    x = _rand_x(67, 192, 3)
    x[5] = 0  # all-zero row
    x[6, 3] = np.float16(np.nan)
    x[7, 9] = np.float16(np.inf)
    x[8] = np.float16(6e-8)  # scale underflows to 0 in fp16 -> rscale = inf
    s_c, s_n = O.c_row_scale(x, clip), O.np_row_scale(x, clip)
    assert np.array_equal(s_c.view(np.uint16), s_n.view(np.uint16))
    q_c, q_n = O.c_quantize_rows(x, s_c), O.np_quantize_rows(x, s_n)
    assert np.array_equal(q_c, q_n)
    assert s_c[5] == np.float16(1.0) and not q_c[5].any()
    assert q_c[6, 3] == 0  # NaN -> 0 (cvt.rni.s32.f32 of NaN)
    assert q_c.min() >= -8 and q_c.max() <= 7


def test_quantizer_matches_emulated_kernels():
    x = _rand_x(40, 128, 4)
    x[3] = 0
    s_emu = E.token_scale_kernel(x, 0.95)
    assert np.array_equal(s_emu.view(np.uint16), O.c_row_scale(x, 0.95).view(np.uint16))


def test_quantizer_closed_form_properties():
    x = _rand_x(64, 256, 5)
    s = O.c_row_scale(x, 1.0)
    q = O.c_quantize_rows(x, s)
    # the absmax element lands on +-7 at clip 1 (scale = fp16(absmax/7) is within
    # 2^-11 relative of absmax/7, so absmax/scale is within 7*(1 +- 2^-11))
    am = np.abs(x.astype(np.float32)).argmax(axis=1)
    assert np.all(np.abs(q[np.arange(64), am]) == 7)
    # scaling a row by a power of two scales the fp16 scale and leaves q unchanged
    x2 = (x.astype(np.float32) * 4).astype(np.float16)
    s2 = O.c_row_scale(x2, 1.0)
    assert np.array_equal(s2.astype(np.float32), s.astype(np.float32) * 4)
    assert np.array_equal(O.c_quantize_rows(x2, s2), q)
    # odd symmetry (at clip 1 nothing saturates, so negation is exact)
    assert np.abs(q).max() == 7
    assert np.array_equal(O.c_quantize_rows((-x.astype(np.float32)).astype(np.float16), s), -q)


def test_quantizer_ties_round_half_even_and_saturate():
    # scale 1.0 exactly: row absmax 7 -> scale_h = 1, rscale = 1, v = x
    x = np.array([[7.0, 0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 3.5, -3.5, 6.5, -6.5, 0.25, 0.75, -7.0, 4.5, 5.5] + [0.0] * 48], np.float16)
    s = O.c_row_scale(x, 1.0)
    assert s[0] == np.float16(1.0)
    q = O.c_quantize_rows(x, s)[0, :16]
    assert q.tolist() == [7, 0, 2, 2, 0, -2, -2, 4, -4, 6, -6, 0, 1, -7, 4, 6]
    # clip < 1 pushes values beyond the grid: saturation to [-8, 7]
    x = np.array([[8.0, -8.0, 7.4, -7.6, 100.0, -100.0] + [0.0] * 58], np.float16)
    q = O.c_quantize_rows(x, np.array([1.0], np.float16))[0, :6]
    assert q.tolist() == [7, -8, 7, -8, 7, -8]


def test_quantizer_brute_force_small_scales():
    """All fp16 x against a few scales, against exact rational arithmetic."""
    from fractions import Fraction

    xs = np.arange(0, 0x7C00, 97, dtype=np.uint16).view(np.float16)
    xs = np.concatenate([xs, -xs])
    for sc in (np.float16(1.0), np.float16(0.1234), np.float16(3.0), np.float16(0.007)):
        rscale = np.float32(1.0) / np.float32(sc)
        q = O.c_quantize_rows(xs[None, :], np.array([sc], np.float16))[0]
        for xv, qv in zip(xs[::13], q[::13]):
            # fp32 product rounded once, then round-half-even to integer, then saturate
            prod = np.float32(xv) * rscale  # numpy fp32 multiply is IEEE
            exact = Fraction(float(prod))
            fl = exact.numerator // exact.denominator
            rem = exact - fl
            r = fl + (1 if rem > Fraction(1, 2) or (rem == Fraction(1, 2) and fl % 2 == 1) else 0)
            assert qv == max(-8, min(7, r))


def test_reference_smoke_formula_agrees_within_tie_noise():
    """The dense formula of the reference's kernel smoke test (unrounded fp32
    scale, true division) must agree except on tie-adjacent elements."""
    x = _rand_x(257, 1536, 0, outliers=False)
    clip = 0.95
    s = O.np_row_scale(x, clip)
    q = O.np_quantize_rows(x, s)
    ascale = np.maximum(np.abs(x.astype(np.float32)).max(axis=1, keepdims=True), 1e-6) / 7 * clip
    q_ref = np.clip(np.rint(x.astype(np.float32) / ascale), -8, 7)
    diff = q.astype(np.int32) - q_ref.astype(np.int32)
    assert np.abs(diff).max() <= 1
    assert (diff != 0).mean() < 2e-3


# ----------------------------------------------------------------- layouts

def test_offset_formulas_c_equals_numpy():
    L = O.lib()
    M, N, K = 300, 256, 192
    off, hi = O.np_act_v1_offsets(M, K)
    h = ctypes.c_int()
    for m in range(0, M, 7):
        for k in range(0, K, 5):
            assert L.vdmq_oracle_act_v1_offset(m, k, K, ctypes.byref(h)) == off[m, k] and h.value == hi[m, k]
    off, hi = O.np_wgt_v1_offsets(N, K)
    for n in range(0, N, 7):
        for k in range(0, K, 5):
            assert L.vdmq_oracle_wgt_v1_offset(n, k, K, ctypes.byref(h)) == off[n, k] and h.value == hi[n, k]
    idx = O.np_wscale_v1_indices(N, K)
    for n in range(0, N, 3):
        for bk in range(K // 64):
            assert L.vdmq_oracle_wscale_v1_index(n, bk, K) == idx[n, bk]
    idx = O.np_ascale_v1_indices(512, K)
    for m in range(0, 512, 3):
        for bk in range(K // 64):
            assert L.vdmq_oracle_ascale_v1_index(m, bk, K) == idx[m, bk]


def test_offsets_are_bijections():
    for (R, K, fn) in ((512, 192, O.np_act_v1_offsets), (256, 192, O.np_wgt_v1_offsets)):
        off, hi = fn(R, K)
        key = off * 2 + hi
        assert np.array_equal(np.sort(key.reshape(-1)), np.arange(R * K))
    assert np.array_equal(np.sort(O.np_wscale_v1_indices(256, 192).reshape(-1)), np.arange(256 * 3))
    assert np.array_equal(np.sort(O.np_ascale_v1_indices(512, 192).reshape(-1)), np.arange(512 * 3))


def test_pack_roundtrip_c_and_numpy():
    rng = np.random.default_rng(6)
    M, N, K = 300, 256, 128
    qa = rng.integers(-8, 8, (M, K), dtype=np.int8)
    qw = rng.integers(-8, 8, (N, K), dtype=np.int8)
    pa = O.c_pack_act_v1(qa)
    assert np.array_equal(pa, O.np_pack_act_v1(qa))
    assert np.array_equal(O.c_unpack_act_v1(pa, M, K), qa)
    assert np.array_equal(O.np_unpack_act_v1(pa, M, K), qa)
    assert not pa.reshape(-1)[O.np_act_v1_offsets(512, K)[0][M:]].any()  # padded rows are zero
    pw = O.c_pack_wgt_v1(qw)
    assert np.array_equal(pw, O.np_pack_wgt_v1(qw))
    assert np.array_equal(O.c_unpack_wgt_v1(pw, N, K), qw)
    ws = rng.random(N).astype(np.float16)
    ps = O.c_pack_wscales_v1(ws, K)
    assert np.array_equal(ps, O.np_pack_wscales_v1(ws, K))
    assert np.array_equal(O.c_unpack_wscales_v1(ps, N, K), ws)
    sa = rng.random(M).astype(np.float16)
    assert np.array_equal(O.c_pack_ascales_v1(sa, K), O.np_pack_ascales_v1(sa, K))


def test_weight_row_concat_is_layout_valid():
    """cat([Wq, Wk, Wv], dim=0) of packed buffers == pack(cat) (attention.py:45-54)."""
    rng = np.random.default_rng(7)
    K = 128
    parts = [rng.integers(-8, 8, (128 * n, K), dtype=np.int8) for n in (1, 2, 1)]
    scales = [rng.random(p.shape[0]).astype(np.float16) for p in parts]
    cat = np.concatenate([O.c_pack_wgt_v1(p) for p in parts], axis=0)
    assert np.array_equal(cat, O.c_pack_wgt_v1(np.concatenate(parts, axis=0)))
    cats = np.concatenate([O.c_pack_wscales_v1(s, K) for s in scales], axis=0)
    assert np.array_equal(cats, O.c_pack_wscales_v1(np.concatenate(scales), K))


def test_layouts_match_emulated_cuda_packers():
    """The closed-form v1 layouts equal what the CUDA packers emit, emulated
    lane by lane with ldmatrix semantics from the PTX ISA."""
    M, N, K = 257, 128, 128
    x = _rand_x(M, K, 8)
    clip = 0.95
    s = O.c_row_scale(x, clip)
    qact_emu, asc_emu = E.act_quantize_per_token_kernel(x, s)
    q = O.c_quantize_rows(x, s)
    assert np.array_equal(qact_emu, O.c_pack_act_v1(q))
    assert np.array_equal(asc_emu.view(np.uint16), O.c_pack_ascales_v1(s, K).view(np.uint16))

    rng = np.random.default_rng(9)
    w = rng.standard_normal((N, K)).astype(np.float16)
    wscale = (np.maximum(np.abs(w.astype(np.float32)).max(axis=1), 1e-6) / 7).astype(np.float16)
    qw_emu, ps_emu = E.weight_quantize_per_channel_kernel(w, wscale)
    qw = O.c_quantize_rows(w, wscale)
    assert np.array_equal(qw_emu, O.c_pack_wgt_v1(qw))
    assert np.array_equal(ps_emu.view(np.uint16), O.c_pack_wscales_v1(wscale, K).view(np.uint16))


# ----------------------------------------------------------- GEMM/epilogue

def test_gemm_numpy_equals_c_integer_loops():
    rng = np.random.default_rng(10)
    qx = rng.integers(-8, 8, (37, 320), dtype=np.int8)
    qw = rng.integers(-8, 8, (48, 320), dtype=np.int8)
    acc = O.c_gemm_i32(qx, qw)
    assert np.array_equal(acc, O.np_gemm_i32(qx, qw))
    assert np.array_equal(acc, qx.astype(np.int64) @ qw.astype(np.int64).T)
    # extreme values: every product 64
    assert O.c_gemm_i32(np.full((1, 14336), -8, np.int8), np.full((1, 14336), -8, np.int8))[0, 0] == 14336 * 64


def test_epilogue_c_equals_numpy_and_float64():
    rng = np.random.default_rng(11)
    acc = rng.integers(-900000, 900000, (33, 64), dtype=np.int32)
    as_h = (rng.random(33) * 2).astype(np.float16)
    ws_h = (1e-3 + 9e-3 * rng.random(64)).astype(np.float16)
    b = (0.02 * rng.standard_normal(64)).astype(np.float16)
    for bias in (None, b):
        y_c = O.c_epilogue(acc, as_h, ws_h, bias)
        y_n = O.np_epilogue(acc, as_h, ws_h, bias)
        assert np.array_equal(y_c.view(np.uint16), y_n.view(np.uint16))
        want = acc.astype(np.float64) * as_h.astype(np.float64)[:, None] * ws_h.astype(np.float64)[None, :]
        if bias is not None:
            want = want + bias.astype(np.float64)
        finite = np.isfinite(y_c.astype(np.float64))
        err = np.abs(y_c.astype(np.float64) - want)[finite]
        # two fp16 roundings (and one fp32 product): within 1.01 fp16 ulp of the exact value
        ulp = np.spacing(np.abs(want[finite]).astype(np.float16)).astype(np.float64)
        assert np.all(err <= 1.01 * np.maximum(ulp, 2.0 ** -24))


def test_whole_kernel_emulation_matches_oracle():
    """End to end: CUDA packers + mma fragments + scale broadcasts + staged
    store, emulated lane by lane, against the logical-domain oracle."""
    M, N, K = 257, 128, 128
    x = _rand_x(M, K, 12)
    rng = np.random.default_rng(13)
    w = rng.standard_normal((N, K)).astype(np.float16)
    wscale = (np.abs(w.astype(np.float32)).max(axis=1) / 7).astype(np.float16)
    bias = rng.standard_normal(N).astype(np.float16)
    clip = 0.95
    s = E.token_scale_kernel(x, clip)
    qact, asc = E.act_quantize_per_token_kernel(x, s)
    qweight, psc = E.weight_quantize_per_channel_kernel(w, wscale)
    y_emu, acc_emu = E.linear_w4a4_kernel(qact, qweight, asc, psc, bias, M, N, K, return_acc=True)

    qw = O.c_quantize_rows(w, wscale)
    y, qx, as_h, acc = O.c_linear(x, qw, wscale, bias, clip)
    assert np.array_equal(acc_emu, acc)
    assert np.array_equal(y_emu.view(np.uint16), y.view(np.uint16))
    y2, _, _, acc2 = O.np_linear(x, qw, wscale, bias, clip)
    assert np.array_equal(acc2, acc) and np.array_equal(y2.view(np.uint16), y.view(np.uint16))

    # and the dense formula the reference's smoke test prints against, to tolerance
    ascale = np.maximum(np.abs(x.astype(np.float32)).max(axis=1, keepdims=True), 1e-6) / 7 * clip
    qx_s = np.clip(np.rint(x.astype(np.float32) / ascale), -8, 7)
    qw_s = np.clip(np.rint(w.astype(np.float32) / wscale.astype(np.float32)[:, None]), -8, 7)
    ref = (qx_s @ qw_s.T) * ascale * wscale.astype(np.float32)[None, :] + bias.astype(np.float32)[None, :]
    rel_l2 = np.linalg.norm(y.astype(np.float32) - ref) / np.linalg.norm(ref)
    assert rel_l2 < 2e-2


# ------------------------------------------------------- committed fixture

def test_oracle_reproduces_the_committed_emulation_fixture():
    """tests/golden/w4a4_emulated_257x128x128.npz was written by the PTX-level
    emulation (tests/golden/make_w4a4_fixture.py); the oracle must reproduce every
    array of it."""
    from pathlib import Path

    f = np.load(Path(__file__).parent / "golden" / "w4a4_emulated_257x128x128.npz")
    x, w, wscale, bias, clip = f["x"], f["w"], f["wscale"], f["bias"], float(f["clip"])
    s = O.c_row_scale(x, clip)
    assert np.array_equal(s.view(np.uint16), f["act_scales"].view(np.uint16))
    q = O.c_quantize_rows(x, s)
    assert np.array_equal(O.c_pack_act_v1(q), f["qact"])
    assert np.array_equal(O.c_pack_ascales_v1(s, 128).view(np.uint16), f["ascales"].view(np.uint16))
    qw = O.c_quantize_rows(w, wscale)
    assert np.array_equal(O.c_pack_wgt_v1(qw), f["qweight"])
    assert np.array_equal(O.c_pack_wscales_v1(wscale, 128).view(np.uint16), f["wscales_packed"].view(np.uint16))
    y, _, _, acc = O.c_linear(x, qw, wscale, bias, clip)
    assert np.array_equal(acc, f["acc"])
    assert np.array_equal(y.view(np.uint16), f["y"].view(np.uint16))


# ------------------------------------------------- property-based (hypothesis)

from hypothesis import given, settings, strategies as st  # noqa: E402


@settings(max_examples=60, deadline=None)
@given(st.integers(1, 40), st.sampled_from([64, 128, 192]), st.integers(0, 2 ** 31 - 1), st.sampled_from([1.0, 0.95, 0.5, 1.7]))
def test_property_quantizer_c_equals_numpy_on_arbitrary_bit_patterns(M, K, seed, clip):
    """Any fp16 bit pattern (NaN payloads, infinities, subnormals included)."""
    rng = np.random.default_rng(seed)
    x = rng.integers(0, 65536, (M, K)).astype(np.uint16).view(np.float16)
    s_c, s_n = O.c_row_scale(x, clip), O.np_row_scale(x, clip)
    assert np.array_equal(s_c.view(np.uint16), s_n.view(np.uint16))
    assert np.array_equal(O.c_quantize_rows(x, s_c), O.np_quantize_rows(x, s_n))


@settings(max_examples=25, deadline=None)
@given(st.integers(1, 3), st.integers(1, 2), st.integers(1, 3), st.integers(0, 2 ** 31 - 1))
def test_property_v1_roundtrip_and_gemm_invariance(mb, nb, kb, seed):
    """pack -> unpack is the identity for both operands, and a GEMM on unpacked
    v1 buffers equals the GEMM on the logical matrices (layout is a bijection)."""
    rng = np.random.default_rng(seed)
    M, N, K = 100 * mb + 3, 128 * nb, 64 * kb
    qa = rng.integers(-8, 8, (M, K), dtype=np.int8)
    qw = rng.integers(-8, 8, (N, K), dtype=np.int8)
    ua = O.np_unpack_act_v1(O.np_pack_act_v1(qa), M, K)
    uw = O.np_unpack_wgt_v1(O.np_pack_wgt_v1(qw), N, K)
    assert np.array_equal(ua, qa) and np.array_equal(uw, qw)
    assert np.array_equal(O.np_gemm_i32(ua, uw), qa.astype(np.int64) @ qw.astype(np.int64).T)


# ----------------------------------------------------------- fused GELU oracle

def test_gelu_oracle_is_pinned_by_torch_float64_and_by_its_identities():
    """np_gelu_tanh_f16 on all 65 536 fp16 patterns: equal to torch's own GELU(approximate="tanh") evaluated in
    float64 and rounded once (a library routine, not a retyped formula); gelu(x) - gelu(-x) = x; special values.
    torch's fp32 evaluation of an fp16 tensor (what the reference runs) is itself only within 3 fp16 ulp of it."""
    import torch

    allh = np.arange(65536, dtype=np.uint16).view(np.float16)
    g = O.np_gelu_tanh_f16(allh)
    t64 = torch.nn.functional.gelu(torch.from_numpy(allh.astype(np.float64)), approximate="tanh").numpy().astype(np.float16)
    both_nan = np.isnan(g) & np.isnan(t64)
    assert np.array_equal(g.view(np.uint16)[~both_nan], t64.view(np.uint16)[~both_nan])
    assert np.array_equal(np.isnan(g), np.isnan(t64))
    x = allh[np.isfinite(allh)].astype(np.float64)
    assert np.abs(O.np_gelu_tanh_f64(x) - O.np_gelu_tanh_f64(-x) - x).max() < 1e-11
    sp = O.np_gelu_tanh_f16(np.array([np.inf, -np.inf, 0.0, 65504.0, -65504.0, 1.0], dtype=np.float16))
    assert sp[0] == np.inf and np.isnan(sp[1]) and sp[2] == 0 and sp[3] == np.float16(65504.0) and sp[4] == 0
    assert sp[5] == np.float16(0.8411919906082768)  # 0.5 * (1 + tanh(sqrt(2/pi) * 1.044715)), worked by hand
    t32 = torch.nn.functional.gelu(torch.from_numpy(allh.astype(np.float32)), approximate="tanh").numpy().astype(np.float16)
    ok = ~(np.isnan(g) | np.isnan(t32))
    ulp = np.abs(g.view(np.int16).astype(np.int32)[ok] - t32.view(np.int16).astype(np.int32)[ok])
    assert ulp.max() <= 3


def test_layer_norm_oracles_are_pinned_by_torch():
    """np_ln_modulate_f16 / np_ln_affine_f16 against torch's own layer_norm (float64) followed by torch's fp16 CPU
    tensor arithmetic -- the operations the reference's block runs (dit_block.py:100), not a retyped formula --
    plus the invariances that fix the statistics: shift and positive-scale invariance of LN, zero mean, unit
    variance."""
    import torch
    import torch.nn.functional as F

    rng = np.random.default_rng(0)
    M, K, eps = 37, 320, 1e-6
    x = (rng.standard_normal((M, K)) * 3 + 1.5).astype(np.float16)
    a = (0.3 * rng.standard_normal((M, K))).astype(np.float16)
    b = (0.5 * rng.standard_normal((M, K))).astype(np.float16)
    h, aux = O.np_ln_modulate_f16(x, a, b, eps)
    assert set(aux) == {"ln", "s1", "p"}
    xt, at, bt = torch.from_numpy(x), torch.from_numpy(a), torch.from_numpy(b)
    ht = F.layer_norm(xt.double(), (K,), None, None, eps).half() * (1 + at) + bt
    assert ht.dtype == torch.float16
    assert np.array_equal(h.view(np.uint16), ht.numpy().view(np.uint16))
    # one vector per 37 rows
    h1, _ = O.np_ln_modulate_f16(x, a[:1], b[:1], eps, rows_per_vec=M)
    ht1 = F.layer_norm(xt.double(), (K,), None, None, eps).half() * (1 + at[:1]) + bt[:1]
    assert np.array_equal(h1.view(np.uint16), ht1.numpy().view(np.uint16))
    ha = O.np_ln_affine_f16(x, a[:1], b[:1], eps, rows_per_vec=M)
    hta = F.layer_norm(xt.double(), (K,), at[0].double(), bt[0].double(), eps).half()
    assert np.array_equal(ha.view(np.uint16), hta.numpy().view(np.uint16))
    n = O.np_layer_norm_f64(x, 0.0)
    assert np.abs(n.mean(axis=1)).max() < 1e-12 and np.abs((n ** 2).mean(axis=1) - 1).max() < 1e-12
    xf = x.astype(np.float64)
    assert np.abs(O.np_layer_norm_f64(4.0 * xf + 8.0, 0.0) - O.np_layer_norm_f64(xf, 0.0)).max() < 1e-12


def test_gated_residual_oracle_equals_torch_fp16_tensor_arithmetic():
    import torch

    rng = np.random.default_rng(1)
    y = (rng.standard_normal((64, 256)) * 3).astype(np.float16)
    y[0, :8] = [65504, -65504, 0, 1e-7, 6e-8, np.inf, -np.inf, np.nan]
    g = rng.standard_normal((2, 256)).astype(np.float16)
    r = (rng.standard_normal((64, 256)) * 5).astype(np.float16)
    want = (torch.from_numpy(r) + torch.from_numpy(y) * torch.from_numpy(g).repeat_interleave(32, dim=0)).numpy()
    got = O.np_gated_residual(y, g, r, rows_per_gate=32)
    both_nan = np.isnan(want) & np.isnan(got)
    assert np.array_equal(got.view(np.uint16)[~both_nan], want.view(np.uint16)[~both_nan])
    assert np.array_equal(np.isnan(got), np.isnan(want))
    assert np.array_equal(O.np_gated_residual(y, None, None).view(np.uint16), y.view(np.uint16))
    want2 = (torch.from_numpy(r) + torch.from_numpy(y)).numpy()
    got2 = O.np_gated_residual(y, None, r)
    ok = ~np.isnan(want2)
    assert np.array_equal(got2.view(np.uint16)[ok], want2.view(np.uint16)[ok])


def test_bf6_decoder_follows_the_format_and_holds_every_int4_value():
    """np_bf6_decode against the E3M2 value table worked by hand (exponent bias 3, 2 mantissa bits, subnormals at
    e = 0, maximum 28): all 32 magnitudes are listed; every integer -8..8 has exactly one code, and so has every q / 16 -- the
    form the operand blocks use."""
    table = [0, 0.0625, 0.125, 0.1875, 0.25, 0.3125, 0.375, 0.4375, 0.5, 0.625, 0.75, 0.875, 1, 1.25, 1.5, 1.75,
             2, 2.5, 3, 3.5, 4, 5, 6, 7, 8, 10, 12, 14, 16, 20, 24, 28]
    codes = np.arange(64)
    vals = O.np_bf6_decode(codes)
    assert np.array_equal(vals[:32], np.array(table, dtype=np.float64))
    assert np.array_equal(vals[32:], -np.array(table, dtype=np.float64))
    for q in range(-8, 9):
        assert (vals == q).sum() == (2 if q == 0 else 1)  # +0 and -0
        # the blocks hold q / 16, whose code is the sign bit and the magnitude as a plain integer
        assert O.np_bf6_decode(np.array([(32 if q < 0 else 0) | abs(q)]))[0] * O.BF6_BLOCK_SCALE == q
    # unpacker: a hand-built block buffer (row r, column k holds ((r + k) % 16) - 8) decodes to itself
    rows, K = 40, 192
    want = (np.add.outer(np.arange(rows), np.arange(K)) % 16 - 8).astype(np.int64)
    enc = {int(v * 16): int(c) for c, v in zip(codes, vals) if float(v * 16).is_integer() and -8 <= v * 16 <= 8 and not (v == 0 and c >= 32)}
    kblocks, panels = (K + 127) // 128 * 2, (rows + 31) // 32 * 4
    buf = np.zeros((panels, kblocks, 384), np.uint8)  # panels of 8 rows; per k-block [h0 16 B x 8][h1 16 B x 8][h0 8 B x 8][h1 8 B x 8]
    for r in range(rows):
        for kb in range(K // 64):
            for h in range(2):
                bits = np.zeros(192, np.uint8)
                for e in range(32):
                    c = enc[int(want[r, 64 * kb + 32 * h + e])]
                    bits[6 * e: 6 * e + 6] = [(c >> i) & 1 for i in range(6)]
                by = np.packbits(bits, bitorder="little")
                a, b = h * 128 + (r % 8) * 16, 256 + h * 64 + (r % 8) * 8
                buf[r // 8, kb, a: a + 16] = by[:16]
                buf[r // 8, kb, b: b + 8] = by[16:]
    assert np.array_equal(O.np_unpack_bf6_blocks(buf.reshape(-1), rows, K), want.astype(np.float64))
