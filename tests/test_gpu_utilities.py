"""The library's measurement utilities (no counterpart in the reference): the plain copy kernel that the traffic
counters are scaled by, the streaming probe that the quantizers' rates are read against, and the MFMA-only probe that
the GEMMs' rates are read against.  Each must move or compute exactly what it claims, or the figures derived from it
mean nothing."""
import ctypes

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def _lib():
    from dsaquant_amd import _lib as L
    from dsaquant_amd.kernels import vdm_w4a4 as v

    assert v.is_available(), v.load_error()
    return L, L.load()


def _stream():
    return torch.cuda.current_stream().cuda_stream


def test_copy_kernel_copies():
    L, lib = _lib()
    g = torch.Generator(device=DEV).manual_seed(1)
    src = torch.randint(0, 256, (3 * 1024 * 1024 + 48,), generator=g, dtype=torch.uint8, device=DEV)
    dst = torch.zeros_like(src)
    L.check(lib.vdmq_copy_u128(src.data_ptr(), dst.data_ptr(), src.numel(), _stream()))
    assert torch.equal(src, dst)
    with pytest.raises(L.VdmqError):
        L.check(lib.vdmq_copy_u128(src.data_ptr(), dst.data_ptr(), 40, _stream()))  # not a multiple of 16 bytes


@pytest.mark.parametrize("reads,writes", [(8, 3), (4, 1), (1, 1), (4, 0)])
def test_stream_probe_reads_and_writes_what_it_says(reads, writes):
    """Wave w reads vectors [w * reads * 64, (w + 1) * reads * 64) of src and writes vectors [w * writes * 64, ...) of
    dst; the value stored proves that every loaded vector arrived (the XOR of the lane's `reads` vectors, plus j in
    every 32-bit word for the j-th store), and nothing beyond threads * writes vectors is written."""
    L, lib = _lib()
    waves = 37
    threads = waves * 64
    g = torch.Generator(device=DEV).manual_seed(reads * 10 + writes)
    src = torch.randint(-2**31, 2**31 - 1, (waves, reads, 64, 4), generator=g, dtype=torch.int32, device=DEV)
    guard = 5
    dst = torch.full((waves * max(writes, 1) + guard, 64, 4), 0x5A5A5A5A, dtype=torch.int32, device=DEV)
    L.check(lib.vdmq_stream_probe(src.data_ptr(), dst.data_ptr(), threads, reads, writes, _stream()))
    torch.cuda.synchronize()
    x = src[:, 0]
    for j in range(1, reads):
        x = x ^ src[:, j]
    got = dst.cpu().numpy()
    want = np.full_like(got, 0x5A5A5A5A)
    xs = x.cpu().numpy().astype(np.int64)
    for j in range(writes):
        want.reshape(-1, 64, 4)[np.arange(waves) * writes + j] = ((xs + j) & 0xFFFFFFFF).astype(np.uint32).view(np.int32)
    assert np.array_equal(got, want)


def test_stream_probe_rejects_what_it_was_not_built_for():
    L, lib = _lib()
    buf = torch.zeros(1 << 16, dtype=torch.uint8, device=DEV)
    with pytest.raises(L.VdmqError):
        L.check(lib.vdmq_stream_probe(buf.data_ptr(), buf.data_ptr(), 64, 5, 2, _stream()))  # no such mix
    with pytest.raises(L.VdmqError):
        L.check(lib.vdmq_stream_probe(buf.data_ptr(), buf.data_ptr(), 100, 4, 1, _stream()))  # not whole waves
    L.check(lib.vdmq_stream_probe(buf.data_ptr(), buf.data_ptr(), 0, 4, 1, _stream()))  # nothing to do


@pytest.mark.parametrize("kind", [0, 1], ids=["int8", "bf6"])
def test_mfma_probe_counts_its_operations(kind):
    """16 MFMAs per iteration and wave, 8 waves per workgroup; one 32 x 32 x 32 int8 instruction is 65 536 operations,
    one 32 x 32 x 64 on 6-bit operands twice that.  With zero operands every accumulator stays zero, so the checksum it
    writes is zero too."""
    L, lib = _lib()
    iters, workgroups = 7, 5
    operands = torch.zeros(int(lib.vdmq_mfma_probe_operand_bytes()), dtype=torch.uint8, device=DEV)
    out = torch.full((workgroups * 512,), 123, dtype=torch.int32, device=DEV)
    ops = ctypes.c_double(0.0)
    L.check(lib.vdmq_mfma_probe(kind, operands.data_ptr(), iters, workgroups, out.data_ptr(), ctypes.byref(ops), _stream()))
    torch.cuda.synchronize()
    per_mfma = 2 * 32 * 32 * (32 if kind == 0 else 64)
    assert ops.value == float(workgroups * 8 * iters * 16 * per_mfma)
    assert int(out.abs().max()) == 0
    with pytest.raises(L.VdmqError):
        L.check(lib.vdmq_mfma_probe(2, operands.data_ptr(), iters, workgroups, out.data_ptr(), ctypes.byref(ops), _stream()))
