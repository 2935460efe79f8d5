// Internal declarations shared by the vdmq translation units (gfx950 only).
#pragma once

#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "vdmq.h"

namespace vdmq {

// Native rows are padded with zero nibbles up to a multiple of this many
// elements; the GEMM consumes K in steps that divide it (128 or 256).
constexpr int kKStep = 256;

constexpr int kWaveSize = 64;

int fail(int code, const char *fmt, ...) __attribute__((format(printf, 2, 3)));
int check_launch(const char *what);
void record_gemm_launch(const vdmq_gemm_launch_info &info); /* what vdmq_last_gemm_launch reports */

inline int64_t k_padded(int64_t K) { return (K + kKStep - 1) / kKStep * kKStep; }
inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }
inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// kernels' host launchers (no argument checking: the extern "C" layer does it)
// fmt: 0 = native int4 rows, 1 = bf6 blocks
int launch_quantize_act(const __half *x, int64_t M, int64_t K, int64_t ldx, float clip, int act, int fmt, uint8_t *qact,
                        __half *scale_h, hipStream_t stream);
int launch_gelu_tanh(const __half *x, __half *y, int64_t n, hipStream_t stream);
// h_out == nullptr: quantize into qact/scale_h; otherwise write the normalised fp16 rows to h_out
int launch_ln_quantize(const __half *x, int64_t M, int64_t K, int64_t ldx, float eps, int ln_mode, const __half *va, const __half *vb,
                       int64_t ldv, int64_t rows_per_vec, float clip, int fmt, uint8_t *qact, __half *scale_h, __half *h_out, int64_t ldh,
                       hipStream_t stream);
int launch_row_scale(const __half *x, int64_t rows, int64_t K, float clip, __half *scale_h, hipStream_t stream);
int launch_quantize_given_scale(const __half *x, const __half *scale_h, int64_t rows, int64_t K, uint8_t *q, hipStream_t stream);
// Optional tail of the GEMM epilogue: out = residual + y * gate (fp16 operations), see vdmq_gemm_w4a4_ex.
struct GemmTail {
    const __half *gate = nullptr;     /* fp16 [*, N], row m uses row m / rows_per_gate */
    int64_t ldg = 0;
    int rows_per_gate = 1;
    const __half *residual = nullptr; /* fp16 [M, N], row stride ldr */
    int64_t ldr = 0;
    // Output split by column blocks (0 = none): element (m, n) goes to out[(n / split_cols) * part_stride + m * ldo +
    // n % split_cols]; split_cols is a multiple of 64, the width of a wave's corner of a tile, so a wave's stores
    // stay inside one part.  Gate and residual keep their [*, N] addressing.
    int split_cols = 0;
    int64_t part_stride = 0;
};

int launch_gemm(const uint8_t *qact, const __half *ascale, const uint8_t *wq, const __half *wscale, const __half *bias,
                void *out, int out_dtype, int32_t *acc_out, int64_t M, int64_t N, int64_t K, int64_t ldo, const GemmTail &tail,
                hipStream_t stream);

// bf6 matrix path (vdmq_bf6.hip)
constexpr int kBf6PanelKb = 384; /* one 64-deep k-block of an 8-row panel of a bf6 operand, bytes */
// Byte offset, in an operand of `kblocks` k-blocks, of the 16-byte (part_b = false) or 8-byte (true) part of the
// 192-bit string that holds row `row`, k = 64 * kb + 32 * h ... + 31.  Rows are stored in panels of eight, a panel
// k-block after k-block, a k-block as [h = 0: 8 rows x 16 B][h = 1: 8 x 16 B][h = 0: 8 x 8 B][h = 1: 8 x 8 B]: what the
// quantizer's eight-row workgroup writes is one contiguous stream, and the GEMM still fetches whole 128-byte lines.
__host__ __device__ __forceinline__ int64_t bf6_piece(int64_t row, int kb, int h, bool part_b, int kblocks) {
    return (row >> 3) * kblocks * kBf6PanelKb + static_cast<int64_t>(kb) * kBf6PanelKb +
           (part_b ? 256 + h * 64 + (row & 7) * 8 : h * 128 + (row & 7) * 16);
}

int64_t bf6_kblocks(int64_t K);
int64_t bf6_bytes(int64_t rows, int64_t K);
int launch_nibbles_to_bf6(const uint8_t *native, int64_t rows, int64_t K, uint8_t *blocks, hipStream_t stream);
int launch_weight_v1_to_bf6(const uint8_t *qweight_v1, int64_t N, int64_t K, uint8_t *blocks, hipStream_t stream);
int launch_bf6_to_weight_v1(const uint8_t *blocks, int64_t N, int64_t K, uint8_t *qweight_v1, hipStream_t stream);
int launch_gemm_bf6(const uint8_t *xblocks, const __half *ascale, const uint8_t *wblocks, const __half *wscale, const __half *bias,
                    void *out, int out_dtype, int32_t *acc_out, int64_t M, int64_t N, int64_t K, int64_t ldo, const GemmTail &tail,
                    hipStream_t stream);

// matrix-pipe ceiling probe (vdmq_probe.hip)
int64_t mfma_probe_operand_bytes();
int launch_mfma_probe(int kind, const void *operands, int iters, int workgroups, void *out, double *ops, hipStream_t stream);

}  // namespace vdmq
