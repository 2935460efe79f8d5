"""Every linear of the benchmark configurations at its full size, on both matrix paths.

Config 1 = Wan-2.1 1.3B at 480p x 81 frames (M = 32760), config 2 = Wan-2.2 5B at 704 x 1280 x 121 frames (M = 27280,
run as the two back-to-back calls of the CFG pair), config 3 = Wan-2.1 14B at 720p (M = 75600; its fused-QKV and
FFN-down shapes are in test_gpu_parity.py, the two others here).  A full-size output cannot go through the CPU oracle
in seconds, so each case checks

* a sample of rows -- the first tile's, some in the middle, the last tile's tail -- against the oracle, bit for bit
  (the contractual bound max|err| <= 1e-3 * max|Y| is asserted too);
* rows are independent: the first 4113 rows of the full run equal a run on those rows alone (another launch
  geometry, other tiles, another tile order);
* which kernel and tile order the library chose, where the choice has special cases: the bf6 path's kernel that walks
  tiles (also where tile rows or columns are left over and regrouped), the one-workgroup-per-tile kernel with
  128 x 128 tiles that small problems take, 16 x 2 super-tiles for six tile columns, contiguous runs for wide N; the
  int8 path's three tile shapes.
"""
import numpy as np
import pytest
import torch

import oracle as O

pytestmark = pytest.mark.gpu

DEV = "cuda:0"

W4, BF6, BF6P = 1, 2, 3  # VDMQ_KERNEL_* of include/vdmq.h

# (config, name, M, K, N, calls, {path: (kernel, tile_m, tile_n, group_n, contiguous)})
CASES = [
    ("cfg1", "qkv", 32760, 1536, 4608, 1, {"int8": (W4, 256, 128, 4, 0), "bf6": (BF6P, 256, 256, 4, 0)}),
    ("cfg1", "o", 32760, 1536, 1536, 1, {"int8": (W4, 256, 128, 4, 0), "bf6": (BF6P, 256, 256, 4, 0)}),       # six tile columns: four as 8 x 4, two as 16 x 2
    ("cfg1", "ffn_up", 32760, 1536, 8960, 1, {"int8": (W4, 256, 256, 4, 0), "bf6": (BF6P, 256, 256, 4, 0)}),
    ("cfg1", "ffn_down", 32760, 8960, 1536, 1, {"int8": (W4, 256, 128, 4, 0), "bf6": (BF6P, 256, 256, 4, 0)}),
    ("cfg1", "cross_kv", 512, 1536, 3072, 1, {"int8": (W4, 128, 128, 4, 0), "bf6": (BF6, 128, 128, 4, 0)}),
    ("cfg2", "qkv", 27280, 3072, 9216, 2, {"int8": (W4, 256, 256, 4, 1), "bf6": (BF6P, 256, 256, 4, 0)}),
    ("cfg2", "o", 27280, 3072, 3072, 2, {"int8": (W4, 256, 256, 4, 1), "bf6": (BF6P, 256, 256, 4, 0)}),
    ("cfg2", "ffn_up", 27280, 3072, 14336, 2, {"int8": (W4, 256, 256, 4, 1), "bf6": (BF6P, 256, 256, 4, 1)}),  # three tile rows left over: regrouped
    ("cfg2", "ffn_down", 27280, 14336, 3072, 2, {"int8": (W4, 256, 256, 4, 1), "bf6": (BF6P, 256, 256, 4, 0)}),
    ("cfg3", "o", 75600, 5120, 5120, 1, {"int8": (W4, 256, 256, 4, 1), "bf6": (BF6P, 256, 256, 4, 0)}),
    ("cfg3", "ffn_up", 75600, 5120, 13824, 1, {"int8": (W4, 256, 256, 4, 1), "bf6": (BF6P, 256, 256, 4, 1)}),
    ("cfg3", "cross_kv", 512, 5120, 10240, 1, {"int8": (W4, 128, 128, 4, 0), "bf6": (BF6, 128, 128, 2, 1)}),
]


def _dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).to(DEV)


def _walks_tiles() -> bool:
    """The bf6 path's tile-walking kernel has one workgroup per CU position of 8 XCDs x 32 CUs and is only taken on a
    device with exactly that many CUs (an MI355X in its default partition mode); elsewhere the launcher uses the
    one-workgroup-per-tile kernel for the same tile order.  (The host-side enumeration of that order,
    tests/tilemap_check.cpp, covers 32 tiles per super-tile, which is what both kernels use.)"""
    return torch.cuda.get_device_properties(DEV).multi_processor_count == 256


def _expected_bf6_kernel(kernel: int) -> int:
    return kernel if _walks_tiles() or kernel != BF6P else BF6


def _activations(M, K, seed):
    """fp16 ~ N(0, 1) with 1 % of the channels scaled by 20, generated on the device (391 M elements at the largest)."""
    g = torch.Generator(device=DEV).manual_seed(seed)
    x = torch.randn((M, K), generator=g, device=DEV, dtype=torch.float16)
    cols = torch.randperm(K, generator=g, device=DEV)[: -(-K // 100)]
    x[:, cols] *= 20
    return x


@pytest.mark.parametrize("path", ["int8", "bf6"])
@pytest.mark.parametrize("cfg,name,M,K,N,calls,expect", CASES, ids=[f"{c[0]}-{c[1]}" for c in CASES])
def test_full_size_linear(cfg, name, M, K, N, calls, expect, path):
    from dsaquant_amd import _lib
    from dsaquant_amd.kernels import vdm_w4a4 as v

    assert v.is_available(), v.load_error()
    _, qw, ws, bias = O.synth_linear(1, K, N, seed=len(name) + K)
    qv1, sv1, b = _dev(O.np_pack_wgt_v1(qw)), _dev(O.np_pack_wscales_v1(ws, K)), _dev(bias)
    old = v.matrix_path()
    v.set_matrix_path(path)
    try:
        for call in range(calls):  # config 2: the cond and the uncond forward, one after the other
            x = _activations(M, K, seed=1000 * call + N)
            print(f"{cfg} {name} M={M} K={K} N={N} path={path} call={call}", flush=True)
            y = v.linear_vdm_w4a4(x, qv1, sv1, b, clip_ratio=1.0)
            info = _lib.last_gemm_launch()
            got_choice = (info.kernel, info.tile_m, info.tile_n, info.group_n, info.contiguous_runs)
            want_choice = (_expected_bf6_kernel(expect[path][0]),) + expect[path][1:]
            assert got_choice == want_choice, f"launcher chose {got_choice}"
            assert y.shape == (M, N) and y.dtype == torch.float16
            rows = np.unique(np.concatenate([np.arange(0, min(M, 40)), np.arange(M // 2, min(M, M // 2 + 24)), np.arange(max(0, M - 40), M)]))
            rows_d = torch.from_numpy(rows).to(DEV)
            want = O.np_linear(x[rows_d].cpu().numpy(), qw, ws, bias, 1.0)[0]
            got = y[rows_d].cpu().numpy()
            err = np.abs(got.astype(np.float32) - want.astype(np.float32)).max()
            assert err <= 1e-3 * np.abs(want.astype(np.float32)).max()
            assert np.array_equal(got.view(np.uint16), want.view(np.uint16))
            P = min(M, 4113)
            y_prefix = v.linear_vdm_w4a4(x[:P], qv1, sv1, b, clip_ratio=1.0)
            assert torch.equal(y[:P], y_prefix)
            torch.cuda.synchronize()
            del x, y, y_prefix
    finally:
        v.set_matrix_path(old)
        torch.cuda.empty_cache()


def test_persistent_bf6_kernel_with_one_to_six_k_steps():
    """The bf6 kernel that walks tiles prefetches the next tile's first two K steps under the epilogue and has
    branches for K of one, two and three steps (K = 64/128, 256, 384); its K loop issues a stage's loads in two halves
    and runs through its step variants in a fixed order that four, five and six steps (K = 512, 640, 768) exercise from
    the first to the last: 65 x 16 tiles, four per workgroup and more, outputs against the int8 path and, for a slice,
    the oracle."""
    from dsaquant_amd import _lib
    from dsaquant_amd.kernels import vdm_w4a4 as v

    assert v.is_available(), v.load_error()
    rng = np.random.default_rng(5)
    M, N = 16400, 4096
    for K in (64, 128, 256, 384, 512, 640, 768):
        qw = rng.integers(-8, 8, (N, K), dtype=np.int8)
        x = O.synth_linear(M, K, 128, seed=K)[0]
        _, _, ws, bias = O.synth_linear(1, 64, N, seed=K + 1)
        print(f"persistent bf6 short K={K}", flush=True)
        old = v.matrix_path()
        try:
            out = {}
            for path in ("bf6", "int8"):
                v.set_matrix_path(path)
                out[path] = v.linear_vdm_w4a4(_dev(x), _dev(O.np_pack_wgt_v1(qw)), _dev(O.np_pack_wscales_v1(ws, K)), _dev(bias), clip_ratio=1.0)
                if path == "bf6":
                    info = _lib.last_gemm_launch()
                    assert info.kernel == _expected_bf6_kernel(BF6P) and (info.workgroups == 256 or not _walks_tiles())
            assert torch.equal(out["bf6"], out["int8"])
            rows = np.r_[0:20, 8190:8210, M - 20:M]
            want = O.np_linear(x[rows], qw, ws, bias, 1.0)[0]
            assert np.array_equal(out["bf6"][torch.from_numpy(rows).to(DEV)].cpu().numpy().view(np.uint16), want.view(np.uint16))
        finally:
            v.set_matrix_path(old)


@pytest.mark.parametrize("M,N,K,group_n,contig", [
    (27280, 14336, 2048, 4, 1),   # three tile rows left over: bottom edge regrouped 3 x 10, contiguous runs of equal length
    (18944 + 100, 13824, 128, 4, 0),  # 54 tile columns: the last two regrouped 16 x 2; a partly filled bottom row as well
    (32760, 4608, 64, 4, 0),      # 18 tile columns: 10 -> 9 rounds with the last two regrouped
    (27280, 35 * 256, 64, 4, 0),  # 107 x 35 tiles: three columns and three rows left over, both regrouped (16 -> 15 rounds)
])
def test_bf6_tile_orders_with_regrouped_edges(M, N, K, group_n, contig):
    """Problems whose tile grid leaves rows or columns over and whose edge super-tiles the launcher regroups: every
    output element against the int8 path (a tile left out or stored twice with other operands would show), sampled
    rows against the oracle, and the launch the library reports."""
    from dsaquant_amd import _lib
    from dsaquant_amd.kernels import vdm_w4a4 as v

    assert v.is_available(), v.load_error()
    rng = np.random.default_rng(M + N + K)
    qw = rng.integers(-8, 8, (N, K), dtype=np.int8)
    x = O.synth_linear(M, K, 128, seed=K)[0]
    _, _, ws, bias = O.synth_linear(1, 64, N, seed=K + 1)
    print(f"regrouped edges M={M} N={N} K={K}", flush=True)
    old = v.matrix_path()
    try:
        out = {}
        for path in ("bf6", "int8"):
            v.set_matrix_path(path)
            out[path] = v.linear_vdm_w4a4(_dev(x), _dev(O.np_pack_wgt_v1(qw)), _dev(O.np_pack_wscales_v1(ws, K)), _dev(bias), clip_ratio=1.0)
            if path == "bf6":
                info = _lib.last_gemm_launch()
                assert (info.kernel, info.group_n, info.contiguous_runs) == (_expected_bf6_kernel(BF6P), group_n, contig)
        assert torch.equal(out["bf6"], out["int8"])
        rows = np.r_[0:8, M // 2:M // 2 + 8, M - 8:M]
        want = O.np_linear(x[rows], qw, ws, bias, 1.0)[0]
        assert np.array_equal(out["bf6"][torch.from_numpy(rows).to(DEV)].cpu().numpy().view(np.uint16), want.view(np.uint16))
    finally:
        v.set_matrix_path(old)
        torch.cuda.empty_cache()


@pytest.mark.parametrize("M,K,N,tile", [
    (300, 192, 384, 128),       # a handful of tiles, ragged M, K of one and a half steps
    (512, 6144 - 128, 3072, 128),  # 47 K steps, 24 big tiles
    (32768, 256, 256, 128),     # exactly 128 big tiles: the last problem that takes small ones; one tile column
    (33024, 256, 256, 256),     # 129 big tiles
    (2048 + 9, 1536, 10240, 256),  # 360 big tiles, too uneven for the tile-walking kernel's fixed places or not: either big kernel
    (128, 64, 128, 128),        # one tile, one k-block
])
def test_bf6_tile_size_follows_the_problem_size(M, K, N, tile):
    """Problems of at most 128 tiles of 256 x 256 (half a tile per CU) run the bf6 GEMM with 128 x 128 tiles, two
    workgroups of four waves per CU; larger ones with 256 x 256.  Every output element against the int8 path, sampled
    rows against the oracle, and the tile size the library reports."""
    from dsaquant_amd import _lib
    from dsaquant_amd.kernels import vdm_w4a4 as v

    assert v.is_available(), v.load_error()
    rng = np.random.default_rng(M + N + K)
    qw = rng.integers(-8, 8, (N, K), dtype=np.int8)
    x = O.synth_linear(M, K, 128, seed=K)[0]
    _, _, ws, bias = O.synth_linear(1, 64, N, seed=K + 1)
    print(f"tile size M={M} K={K} N={N}", flush=True)
    old = v.matrix_path()
    try:
        out = {}
        for path in ("bf6", "int8"):
            v.set_matrix_path(path)
            out[path] = v.linear_vdm_w4a4(_dev(x), _dev(O.np_pack_wgt_v1(qw)), _dev(O.np_pack_wscales_v1(ws, K)), _dev(bias), clip_ratio=1.0)
            if path == "bf6":
                info = _lib.last_gemm_launch()
                assert (info.tile_m, info.tile_n) == (tile, tile), f"launcher chose {info.tile_m} x {info.tile_n}"
                assert info.kernel == BF6 if tile == 128 else info.kernel in (BF6, BF6P)
        assert torch.equal(out["bf6"], out["int8"])
        rows = np.unique(np.r_[0:min(M, 8), M // 2:min(M, M // 2 + 8), max(0, M - 8):M])
        want = O.np_linear(x[rows], qw, ws, bias, 1.0)[0]
        assert np.array_equal(out["bf6"][torch.from_numpy(rows).to(DEV)].cpu().numpy().view(np.uint16), want.view(np.uint16))
    finally:
        v.set_matrix_path(old)
        torch.cuda.empty_cache()
