"""The entry point that allocates nothing, vdmq_linear_w4a4_noalloc, called raw through the C ABI.

Its workspace is a buffer built into the library's device code, so the test checks what matters about that: the
output is the same bits as vdmq_linear_w4a4 with a caller workspace (and as the oracle's), on two calls in a row that
share the buffer -- the second with a smaller input, which finds the first call's contents there."""
import ctypes

import numpy as np
import pytest
import torch

import oracle as O

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def _pack_native(q: np.ndarray, Kp: int) -> np.ndarray:
    R, K = q.shape
    full = np.zeros((R, Kp), np.uint8)
    full[:, :K] = q.astype(np.uint8) & 0xF
    return (full[:, 0::2] | (full[:, 1::2] << 4)).astype(np.uint8)


def _dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).to(DEV)


def _run_pair(lib, check, M, K, N, seed, clip, use_bias):
    x, qw, ws, bias = O.synth_linear(M, K, N, seed=seed)
    Kp = int(lib.vdmq_k_padded(K))
    xd, wd, sd = _dev(x), _dev(_pack_native(qw, Kp)), _dev(ws)
    bd = _dev(bias) if use_bias else None
    bias_p = bd.data_ptr() if use_bias else None
    stream = torch.cuda.current_stream().cuda_stream
    out_ws = torch.full((M, N), float("nan"), dtype=torch.float16, device=DEV)
    out_na = torch.full((M, N), float("nan"), dtype=torch.float16, device=DEV)
    work = torch.empty(int(lib.vdmq_workspace_bytes(M, K)), dtype=torch.uint8, device=DEV)
    print(f"no-alloc linear M={M} K={K} N={N} clip={clip} bias={use_bias}", flush=True)
    check(lib.vdmq_linear_w4a4(xd.data_ptr(), M, K, K, clip, wd.data_ptr(), sd.data_ptr(), bias_p, out_ws.data_ptr(), 0, N, N,
                               work.data_ptr(), work.numel(), stream))
    # a first call, outside the measured window: the one-time look-up of the built-in buffer's address and the kernels'
    # LDS-size attributes happen here
    check(lib.vdmq_linear_w4a4_noalloc(xd.data_ptr(), M, K, K, clip, wd.data_ptr(), sd.data_ptr(), bias_p, out_na.data_ptr(), 0, N, N, stream))
    torch.cuda.synchronize()
    out_na.fill_(float("nan"))
    torch.cuda.synchronize()
    # "allocates nothing" as the driver sees it: the device's free memory (torch's own counters would only show
    # allocations made through torch's allocator, which a hipMalloc inside the library bypasses)
    free_before, torch_before = torch.cuda.mem_get_info()[0], torch.cuda.memory_reserved()
    check(lib.vdmq_linear_w4a4_noalloc(xd.data_ptr(), M, K, K, clip, wd.data_ptr(), sd.data_ptr(), bias_p, out_na.data_ptr(), 0, N, N, stream))
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before and torch.cuda.memory_reserved() == torch_before
    want = O.np_linear(x, qw, ws, bias if use_bias else None, clip)[0]
    got = out_na.cpu().numpy()
    assert np.array_equal(got.view(np.uint16), out_ws.cpu().numpy().view(np.uint16))  # same bits as the entry point it is a variant of
    assert np.array_equal(got.view(np.uint16), want.view(np.uint16))                  # and as the oracle


def test_noalloc_linear_twice_second_call_smaller():
    from dsaquant_amd import _lib

    lib = _lib.load()
    _run_pair(lib, _lib.check, 1000, 1536, 1536, seed=41, clip=0.95, use_bias=True)
    _run_pair(lib, _lib.check, 300, 512, 256, seed=42, clip=1.0, use_bias=False)   # smaller: the buffer holds the first call's rows
    _run_pair(lib, _lib.check, 2049, 3072, 128, seed=43, clip=1.0, use_bias=True)  # and larger again, on the 128 x 128 tiles


def test_noalloc_refuses_inputs_beyond_its_buffer():
    from dsaquant_amd import _lib

    lib = _lib.load()
    x = torch.zeros((8, 64), dtype=torch.float16, device=DEV)
    M, K = 75600, 5120  # 194 MB of quantized rows
    assert lib.vdmq_workspace_bytes(M, K) > 64 << 20
    rc = lib.vdmq_linear_w4a4_noalloc(x.data_ptr(), M, K, K, 1.0, x.data_ptr(), x.data_ptr(), None, x.data_ptr(), 0, 128, 128, None)
    assert rc == -4 and b"scratch" in lib.vdmq_last_error()
    torch.cuda.synchronize()
    # the largest config-1 and config-2 activations fit
    for m, k in ((32760, 1536), (27280, 3072), (512, 5120)):
        assert lib.vdmq_workspace_bytes(m, k) <= 64 << 20
