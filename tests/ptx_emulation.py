"""Thread-by-thread emulation of the reference's CUDA packers and GEMM kernel.

Test helper, independent of the closed-form offset formulas in ``oracle/``:
it walks the kernels of ``vdm_infer/kernels/csrc/vdm_w4a4_kernel.cu`` lane by
lane (32-lane warps) and implements the PTX instructions they use from the
PTX ISA's own definitions:

* ``cvt.rni.s32.f32`` -- round to nearest even, NaN -> 0.
* ``cvt.pack.sat.s4.s32.b32 d, a, b, c`` -- d = (c << 8) | (sat4(a) << 4) | sat4(b).
* ``ldmatrix.sync.aligned.x4.m8n8.shared.b16`` -- lanes 8j..8j+7 give the row
  addresses of matrix j; lane t receives, from each matrix, the 32-bit word
  (two b16) at row t/4, word t%4.
* ``mma.sync.aligned.m16n8k64.row.col.s32.s4.s4.s32`` -- fragment layouts of
  the PTX ISA "Matrix Fragments for mma.m16n8k64" section (g = lane/4, t = lane%4):
    A: a0 (row g,   k 8t..8t+7), a1 (row g+8, k 8t..8t+7),
       a2 (row g,   k 32+8t..),  a3 (row g+8, k 32+8t..)
    B: b0 (k 8t..8t+7, col g),   b1 (k 32+8t.., col g)
    C: c0 (g, 2t), c1 (g, 2t+1), c2 (g+8, 2t), c3 (g+8, 2t+1)
  element e of a register is its nibble e (bits 4e..4e+3), two's complement.

Pure numpy/Python loops: use small shapes only.
"""
from __future__ import annotations

import numpy as np

BLOCK_M, BLOCK_N, WARP_K, NUM_WARPS = 256, 128, 64, 8


def _rni(v: np.float32) -> int:
    if np.isnan(v):
        return 0
    if v >= 2147483647.0:
        return 2147483647
    if v <= -2147483648.0:
        return -2147483648
    return int(np.rint(v))


def _sat4(v: int) -> int:
    return max(-8, min(7, v)) & 0xF


def quantize_float2_s4(x: np.float32, y: np.float32) -> int:
    """.cu:95-102: cvt.pack with a = rni(y), b = rni(x)."""
    v1, v2 = _rni(x), _rni(y)
    return (_sat4(v2) << 4) | _sat4(v1)


def _ldmatrix_x4(mat: np.ndarray, lane_addr):
    """mat: u32[16][8]; lane_addr[l] = (row, word) supplied by lane l.
    Returns u32[32][4]."""
    out = np.zeros((32, 4), np.uint32)
    for t in range(32):
        for j in range(4):
            row, word = lane_addr[8 * j + t // 4]
            out[t, j] = mat[row, word + t % 4]
    return out


def quantize_warp_static_scale(inp: np.ndarray, scales: np.ndarray):
    """.cu:296-338 (and the guarded twin :341-393 once the caller has zeroed
    invalid rows and set their scale to 1).  inp: fp16 [16, 64]; scales fp16 [16].
    Returns (u32[32][4] fragment words per lane, fp16[16] output scales)."""
    mat = np.zeros((16, 8), np.uint32)
    oscale = np.zeros(16, np.float16)
    for i in range(4):
        for lane in range(32):
            row_id = i * 4 + lane // 8
            col_id = (lane % 8) * 8
            pack = inp[row_id, col_id:col_id + 8]
            scale_f = np.float32(scales[row_id])
            with np.errstate(divide="ignore"):
                rscale = np.float32(1.0) / scale_f
            if lane % 8 == 0:
                oscale[row_id] = np.float16(scale_f)
            qpack = 0
            for j in range(0, 8, 2):
                with np.errstate(invalid="ignore", over="ignore"):
                    fx = np.float32(pack[j]) * rscale
                    fy = np.float32(pack[j + 1]) * rscale
                qpack |= quantize_float2_s4(fx, fy) << (j * 4)
            mat[row_id, lane % 8] = qpack
    lane_addr = [(lane % 16, lane // 16 * 4) for lane in range(32)]
    return _ldmatrix_x4(mat, lane_addr), oscale


def token_scale_kernel(x: np.ndarray, clip: float) -> np.ndarray:
    """.cu:459-481, with the 256-thread strided loop and the tree reduction."""
    M, K = x.shape
    out = np.zeros(M, np.float16)
    for row in range(M):
        smem = np.zeros(256, np.float32)
        for tid in range(256):
            vals = np.abs(x[row, tid:K:256].astype(np.float32))
            local = np.float32(0.0)
            for v in vals:
                local = np.fmax(local, v)
            smem[tid] = local
        stride = 128
        while stride > 0:
            smem[:stride] = np.fmax(smem[:stride], smem[stride:2 * stride])
            stride >>= 1
        scale = (smem[0] / np.float32(7.0)) * np.float32(clip) if smem[0] > 0 else np.float32(1.0)
        out[row] = np.float16(scale)
    return out


def act_quantize_per_token_kernel(x: np.ndarray, token_scales: np.ndarray):
    """.cu:483-516.  Returns (qact u8 [paddedM, K/2], ascales fp16 [paddedM, K/64])."""
    M, K = x.shape
    PM = (M + BLOCK_M - 1) // BLOCK_M * BLOCK_M
    KG = K // WARP_K
    out_words = np.zeros((PM * K // 2) // 16 * 4, np.uint32).reshape(-1, 4)  # uint4 array
    oscales = np.zeros(PM * KG, np.float16).reshape(-1, 2)  # packed_ascale_t = one half2
    for bx in range(PM // 32):
        for bk in range(KG):
            bm, warp_id = bx // 8, bx % 8
            row, col = bx * 32, bk * WARP_K
            oscale_shmem = np.zeros(32, np.float16)
            for tile_id in range(2):
                tile_row = row + tile_id * 16
                inp = np.zeros((16, 64), np.float16)
                sc = np.ones(16, np.float16)
                for r in range(16):
                    if tile_row + r < M:
                        inp[r] = x[tile_row + r, col:col + 64]
                        sc[r] = token_scales[tile_row + r]
                frag, osc = quantize_warp_static_scale(inp, sc)
                oscale_shmem[tile_id * 16:(tile_id + 1) * 16] = osc
                base = (((bm * KG + bk) * NUM_WARPS + warp_id) * 2 + tile_id) * 32
                out_words[base:base + 32] = frag
            # pack_ascales .cu:276-284
            obase = ((bm * KG + bk) * NUM_WARPS + warp_id) * 16
            for lane in range(16):
                a = oscale_shmem[lane // 8 * 16 + lane % 8]
                b = oscale_shmem[lane // 8 * 16 + lane % 8 + 8]
                oscales[obase + lane] = (a, b)
    qact = out_words.reshape(-1).view(np.uint8).reshape(PM, K // 2)
    return qact, oscales.reshape(PM, KG)


def weight_quantize_per_channel_kernel(w: np.ndarray, channel_scales: np.ndarray):
    """.cu:518-551.  Returns (qweight u8 [N, K/2], packed scales fp16 [N, K/64])."""
    N, K = w.shape
    KG = K // WARP_K
    out_words = np.zeros((N * K // 2) // 16 * 4, np.uint32).reshape(-1, 4)
    pscales = np.zeros(N * KG, np.float16).reshape(-1, 4)  # packed_wscale_t = four halves
    for bn in range(N // BLOCK_N):
        for bk in range(KG):
            col, row = bn * BLOCK_N, bk * WARP_K
            oscale_shmem = np.zeros(128, np.float16)
            for tile_id in range(8):
                n0 = col + tile_id * 16
                frag, osc = quantize_warp_static_scale(w[n0:n0 + 16, row:row + 64], channel_scales[n0:n0 + 16])
                oscale_shmem[tile_id * 16:(tile_id + 1) * 16] = osc
                frag = frag[:, [0, 2, 1, 3]]  # swap .y/.z, .cu:542-544
                base = ((bn * KG + bk) * 8 + tile_id) * 32
                out_words[base:base + 32] = frag
            # pack_wscales .cu:286-294
            obase = (bn * KG + bk) * 32
            for lane in range(32):
                for i in (0, 2):
                    src = lane // 4 * 16 + lane % 4 * 2 + i * 4
                    pscales[obase + lane, i:i + 2] = oscale_shmem[src:src + 2]
    qweight = out_words.reshape(-1).view(np.uint8).reshape(N, K // 2)
    return qweight, pscales.reshape(N, KG)


def _nibbles(word: int):
    vals = [(int(word) >> (4 * e)) & 0xF for e in range(8)]
    return [v - 16 if v >= 8 else v for v in vals]


def _mma_m16n8k64(a_regs: np.ndarray, b_regs: np.ndarray) -> np.ndarray:
    """a_regs u32[32][4], b_regs u32[32][2] -> c s32[32][4] (zero C input)."""
    A = np.zeros((16, 64), np.int64)
    B = np.zeros((64, 8), np.int64)
    for lane in range(32):
        g, t = lane // 4, lane % 4
        for reg, (row, k0) in enumerate([(g, 8 * t), (g + 8, 8 * t), (g, 32 + 8 * t), (g + 8, 32 + 8 * t)]):
            A[row, k0:k0 + 8] = _nibbles(a_regs[lane, reg])
        for reg, k0 in enumerate([8 * t, 32 + 8 * t]):
            B[k0:k0 + 8, g] = _nibbles(b_regs[lane, reg])
    C = A @ B
    out = np.zeros((32, 4), np.int64)
    for lane in range(32):
        g, t = lane // 4, lane % 4
        out[lane] = (C[g, 2 * t], C[g, 2 * t + 1], C[g + 8, 2 * t], C[g + 8, 2 * t + 1])
    return out


def linear_w4a4_kernel(qact, qweight, ascales, wscales, bias, M, N, K, return_acc=False):
    """.cu:627-686 with finalize_int_accum (:243-274) and store_fpsum (:571-625)."""
    PM = qact.shape[0]
    KG = K // WARP_K
    act = qact.reshape(-1).view(np.uint32).reshape(-1, 4)
    wgt = qweight.reshape(-1).view(np.uint32).reshape(-1, 4)
    asc = ascales.reshape(-1, 2)
    wsc = wscales.reshape(-1, 4)
    out = np.zeros((M, N), np.float16)
    acc_out = np.zeros((M, N), np.int64)
    for bm in range(PM // BLOCK_M):
        for bn in range(N // BLOCK_N):
            act_block = bm * KG * NUM_WARPS * 2 * 32
            wgt_block = bn * KG * 8 * 32
            ascale_block = bm * KG * NUM_WARPS * 16
            wscale_block = bn * KG * 32
            for warp_id in range(NUM_WARPS):
                ipsum = np.zeros((2, 8, 32, 8), np.int64)  # [i][j][lane][8]
                for kg in range(KG):
                    A = [act[act_block + ((kg * NUM_WARPS + warp_id) * 2 + i) * 32:][:32] for i in range(2)]
                    W = [wgt[wgt_block + (kg * 8 + j) * 32:][:32] for j in range(8)]
                    for j in range(8):
                        for i in range(2):
                            o1 = _mma_m16n8k64(A[i], W[j][:, 0:2])
                            o2 = _mma_m16n8k64(A[i], W[j][:, 2:4])
                            ipsum[i, j, :, 0:4] += o1
                            ipsum[i, j, :, 4:8] += o2
                # scales of k-group 0 only, .cu:661-663
                ascale0 = [asc[ascale_block + (0 * NUM_WARPS + warp_id) * 16 + lane] if lane < 16 else None for lane in range(32)]
                wscale0 = [wsc[wscale_block + lane] for lane in range(32)]
                fpsum = np.zeros((2, 8, 32, 4, 2), np.float16)
                for lane in range(32):
                    for i in range(2):
                        a_pair = ascale0[8 * i + lane // 4]  # broadcast_ascale(k = 2i)
                        asx, asy = np.float32(a_pair[0]), np.float32(a_pair[1])
                        for j in range(8):
                            src = wscale0[4 * j + lane % 4]  # broadcast_wscale(k = 4j, 4j+2)
                            ws1 = (np.float32(src[0]), np.float32(src[1]))
                            ws2 = (np.float32(src[2]), np.float32(src[3]))
                            p = ipsum[i, j, lane]

                            def sc(x, y, s0, s1):
                                return (np.float16(np.float32(x) * s0), np.float16(np.float32(y) * s1))

                            fpsum[i, j, lane, 0] = sc(p[0], p[1], asx * ws1[0], asx * ws1[1])
                            fpsum[i, j, lane, 1] = sc(p[2], p[3], asy * ws1[0], asy * ws1[1])
                            fpsum[i, j, lane, 2] = sc(p[4], p[5], asx * ws2[0], asx * ws2[1])
                            fpsum[i, j, lane, 3] = sc(p[6], p[7], asy * ws2[0], asy * ws2[1])
                # store_fpsum
                for i in range(2):
                    for phase, (d_lo, d_hi) in enumerate([(0, 2), (1, 3)]):
                        mat = np.zeros((8, 136), np.float16)
                        accm = np.zeros((8, 136), np.int64)
                        for j in range(8):
                            for lane in range(32):
                                row, col = lane // 4, lane % 4 * 2 + j * 16
                                mat[row, col:col + 2] = fpsum[i, j, lane, d_lo]
                                mat[row, col + 8:col + 10] = fpsum[i, j, lane, d_hi]
                                p = ipsum[i, j, lane]
                                accm[row, col:col + 2] = p[2 * d_lo:2 * d_lo + 2]
                                accm[row, col + 8:col + 10] = p[2 * d_hi:2 * d_hi + 2]
                        for row in range(8):
                            gm = bm * BLOCK_M + warp_id * 32 + i * 16 + phase * 8 + row
                            for lane in range(32):
                                gn = bn * BLOCK_N + lane * 4
                                if gm < M and gn + 3 < N:
                                    pack = mat[row, lane * 4:lane * 4 + 4]
                                    if bias is not None:
                                        # __hadd2: one fp16 addition per element
                                        pack = (pack.astype(np.float64) + bias[gn:gn + 4].astype(np.float64)).astype(np.float16)
                                    out[gm, gn:gn + 4] = pack
                                    acc_out[gm, gn:gn + 4] = accm[row, lane * 4:lane * 4 + 4]
    if return_acc:
        return out, acc_out
    return out
