/*
 * vdmq -- C ABI of the MI355X (gfx950) W4A4 linear hot path.
 *
 * Every entry point takes plain device pointers, sizes and a HIP stream, and
 * returns 0 on success or a negative VDMQ_E* code; vdmq_last_error() then
 * holds a message (thread-local).  No entry point allocates, frees or
 * synchronises: all buffers are caller-owned device memory, all work is
 * enqueued asynchronously on `stream` (0 = the null stream) of the current
 * device.
 *
 * The functions replace the six pybind entry points of the reference
 * extension (vdm_infer/kernels/csrc/vdm_w4a4_kernel.cu:924-940) and the kernel
 * launches behind them; the citation on each declaration names the part it
 * stands in for.  Four utilities with no counterpart there live in the same
 * library, so that measurements and the product come from one build:
 * vdmq_copy_u128 (a plain copy), vdmq_stream_probe (a fixed mix of streamed
 * reads and writes), vdmq_mfma_probe (a loop of matrix instructions only) and
 * vdmq_last_gemm_launch (which kernel and tile order the launcher chose).
 *
 * Layouts
 *   "v1"      the byte order the reference's CUDA packers emit and packed
 *             checkpoints (format "vdm_w4a4_packed_v1") store:
 *             qweight u8 [N, K/2], packed scales fp16 [N, K/64],
 *             qact u8 [ceil(M,256), K/2], ascales fp16 [ceil(M,256), K/64].
 *   "native"  what the gfx950 kernels consume: row-major packed int4,
 *             u8 [rows, Kp/2] with Kp = vdmq_k_padded(K); byte j of a row holds
 *             element 2j in its low nibble and 2j+1 in its high nibble (two's
 *             complement); elements K..Kp-1 are zero.  Scales are one fp16 per
 *             row ([M] for tokens, [N] for output channels).
 */
#ifndef VDMQ_H
#define VDMQ_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define VDMQ_OK 0
#define VDMQ_EINVAL (-1)  /* null pointer, misaligned pointer, bad enum */
#define VDMQ_ESHAPE (-2)  /* a shape precondition failed (K % 64, N % 128, ...) */
#define VDMQ_ELAUNCH (-3) /* the HIP runtime refused a launch */
#define VDMQ_ENOSPACE (-4) /* caller workspace too small */

#define VDMQ_OUT_F16 0
#define VDMQ_OUT_BF16 1

/* elementwise activation applied to the input of a quantizer */
#define VDMQ_ACT_NONE 0
#define VDMQ_ACT_GELU_TANH 1

/* what follows the LayerNorm fused in front of a quantizer */
#define VDMQ_LN_MODULATE 1 /* fp16(LN(x)) * (1 + scale) + shift, fp16 arithmetic */
#define VDMQ_LN_AFFINE 2   /* fp16(LN(x) * weight + bias), fp32 arithmetic */

/* Shape constants of the v1 layout (vdm_w4a4_kernel.cu:15-24, vdm_w4a4.py:23-25). */
#define VDMQ_BLOCK_M 256
#define VDMQ_BLOCK_N 128
#define VDMQ_WARP_K 64

typedef void *vdmq_stream_t; /* hipStream_t */

/* Version of this interface AND of the bf6 block format below: 2 = blocks hold q / 16 (code sign << 5 | |q|).  A host
 * compares vdmq_version() with the VDMQ_VERSION it was compiled against before it hands the library blocks it kept. */
#define VDMQ_VERSION 2
int vdmq_version(void);
const char *vdmq_arch(void);       /* "gfx950" */
const char *vdmq_last_error(void); /* message of the last failure on this thread */

/* Native row length in elements for a logical K (K rounded up to the GEMM's
 * K step).  Native rows are vdmq_k_padded(K)/2 bytes. */
int64_t vdmq_k_padded(int64_t K);

/* Dynamic per-token A4 quantizer.  Replaces token_scale_kernel +
 * act_quantize_per_token_kernel (vdm_w4a4_kernel.cu:459-516, launched at
 * :802-816 and :858-872) with one pass over x.
 *   x       fp16 [M, K], row stride ldx elements (ldx % 8 == 0, 16-byte aligned)
 *   qact    u8 [M, Kp/2] native, 16-byte aligned
 *   scale_h fp16 [M]: fp16_rn(absmax > 0 ? (absmax / 7) * clip : 1)
 * Preconditions: K % 64 == 0, M >= 0. */
int vdmq_quantize_act(const void *x, int64_t M, int64_t K, int64_t ldx, float clip, void *qact, void *scale_h,
                      vdmq_stream_t stream);

/* The same quantizer with the preceding elementwise activation fused in:
 * row m is act(x[m, :]) evaluated in fp32 and rounded once to fp16, then
 * quantized as above.  VDMQ_ACT_GELU_TANH is the FeedForward activation
 * between the two FFN linears (activation_fn="gelu-approximate",
 * vdm_infer/models/wan_vdm/modules/dit_block.py:56):
 *   gelu(x) = 0.5 * x * (1 + tanh(sqrt(2/pi) * (x + 0.044715 * x^3))).
 * Fusing it removes the activation kernel, its [M, K] fp16 write and the
 * quantizer's re-read (the reference runs them separately: FeedForward ->
 * QuantLinear.forward, quant_linear.py:162-172).  The fp16 activation values
 * are those vdmq_gelu_tanh_f16 returns; given them, qact and scale_h are
 * exactly vdmq_quantize_act's. */
int vdmq_quantize_act_ex(const void *x, int64_t M, int64_t K, int64_t ldx, float clip, int act, void *qact, void *scale_h,
                         vdmq_stream_t stream);

/* y[i] = fp16_rn(gelu_tanh(float(x[i]))) for n fp16 values (n even, 4-byte
 * aligned pointers): the activation of vdmq_quantize_act_ex on its own. */
int vdmq_gelu_tanh_f16(const void *x, void *y, int64_t n, vdmq_stream_t stream);

/* The quantizer with the preceding LayerNorm (+ modulation) fused in: the
 * producer of a Wan block's attn1 and FFN-up inputs,
 *   norm(hidden_states) * (1 + scale) + shift
 * (vdm_infer/models/wan_vdm/modules/dit_block.py:100, :110; norm = FP32LayerNorm
 * without affine: statistics in fp32, result cast to fp16), or of the attn2 query
 * input, norm2 with elementwise affine (:105).  Row m of x [M, K] is normalised
 * over K (biased variance, eps inside the square root), then
 *   VDMQ_LN_MODULATE: h = fp16(fp16(fp16(LN) * fp16(1 + a)) + b)   a = scale, b = shift
 *   VDMQ_LN_AFFINE:   h = fp16(LN * a + b) in fp32                 a = weight, b = bias
 * with a, b fp16 [*, K] (row stride ldv elements, ldv % 8 == 0, 16-byte
 * aligned); row m uses vector row m / rows_per_vec (one vector per batch element:
 * rows_per_vec = tokens per batch element; one per token: 1).  h is then
 * quantized as vdmq_quantize_act does.  K <= 16384.
 * vdmq_ln_f16 writes h itself (fp16 [M, K], row stride ldh) with the same
 * arithmetic; given its h, qact and scale_h are exactly vdmq_quantize_act's. */
int vdmq_quantize_act_ln(const void *x, int64_t M, int64_t K, int64_t ldx, float eps, int ln_mode, const void *a, const void *b,
                         int64_t ldv, int64_t rows_per_vec, float clip, void *qact, void *scale_h, vdmq_stream_t stream);
int vdmq_ln_f16(const void *x, int64_t M, int64_t K, int64_t ldx, float eps, int ln_mode, const void *a, const void *b, int64_t ldv,
                int64_t rows_per_vec, void *h, int64_t ldh, vdmq_stream_t stream);

/* W4A4 GEMM with fused epilogue.  Replaces linear_w4a4_kernel
 * (vdm_w4a4_kernel.cu:627-686, launched at :819 and :907):
 *   acc[m,n] = sum_k qact[m,k] * wq[n,k]                      (int32, exact)
 *   out[m,n] = fp16_rn(float(acc) * (float(ascale[m]) * float(wscale[n])))
 *              then, with a bias, one more fp16 addition of bias[n]
 *   qact u8 [M, Kp/2] native; ascale fp16 [M]; wq u8 [N, Kp/2] native;
 *   wscale fp16 [N]; bias fp16 [N] or NULL; out [M, N] with row stride ldo
 *   elements (ldo % 8 == 0, ldo <= 4194304), out_dtype VDMQ_OUT_F16 or VDMQ_OUT_BF16.
 * Preconditions: K % 64 == 0, N % 128 == 0, K <= 65536. */
int vdmq_gemm_w4a4(const void *qact, const void *ascale, const void *wq, const void *wscale, const void *bias, void *out,
                   int out_dtype, int64_t M, int64_t N, int64_t K, int64_t ldo, vdmq_stream_t stream);

/* The same GEMM with the block's gated residual update folded into the
 * epilogue (vdm_infer/models/wan_vdm/modules/dit_block.py:102, :107, :112:
 * hidden_states = hidden_states + attn_output * gate), y being the output of
 * vdmq_gemm_w4a4 (bias included):
 *   out[m,n] = fp16(residual[m,n] + fp16(y[m,n] * gate[m / rows_per_gate, n]))
 * -- the two fp16 tensor operations the reference runs as separate kernels,
 * each correctly rounded.  gate fp16 [*, N] (row stride ldg) or NULL (no
 * multiplication: the attn2 update); residual fp16 [M, N] (row stride ldr) or
 * NULL; `out` may be `residual` itself (in-place update).  16-byte aligned,
 * strides multiples of 8; fp16 output only. */
int vdmq_gemm_w4a4_ex(const void *qact, const void *ascale, const void *wq, const void *wscale, const void *bias, const void *gate,
                      int64_t ldg, int64_t rows_per_gate, const void *residual, int64_t ldr, void *out, int out_dtype, int64_t M,
                      int64_t N, int64_t K, int64_t ldo, vdmq_stream_t stream);

/* vdmq_gemm_w4a4 (fp16 output) writing its N columns as N / split_cols separate matrices: element (m, n) goes to
 *   out[(n / split_cols) * part_stride + m * ldo + n % split_cols]        (fp16 elements)
 * -- the same values vdmq_gemm_w4a4 writes to out[m * ldo + n].  For the fused QKV projection (N = 3 * dim, the
 * reference splits one [M, 3 * dim] result into strided views and unflattens them per head,
 * vdm_infer/kernels/vdm_w4a4.py:297-298, vdm_infer/models/wan_vdm/modules/attention.py:165-172):
 *   split_cols = dim, ldo = dim, part_stride = M * dim        q, k, v as three contiguous [M, dim] matrices
 *   split_cols = head_dim, ldo = head_dim, part_stride = M * head_dim
 *                                                           head-major: [3 * heads][M][head_dim]
 * split_cols is a multiple of 64 that divides N; ldo >= split_cols, ldo and part_stride multiples of 8. */
int vdmq_gemm_w4a4_split(const void *qact, const void *ascale, const void *wq, const void *wscale, const void *bias, void *out, int64_t M,
                         int64_t N, int64_t K, int64_t ldo, int64_t split_cols, int64_t part_stride, vdmq_stream_t stream);

/* Same GEMM, but writes the raw int32 accumulators acc [M, N] (row stride N)
 * instead of the scaled output: the checker's view of the value the reference
 * holds in `ipsum` before finalize_int_accum (vdm_w4a4_kernel.cu:650, :684). */
int vdmq_gemm_w4a4_acc(const void *qact, const void *wq, int32_t *acc, int64_t M, int64_t N, int64_t K, vdmq_stream_t stream);

/* What the library chose for the last GEMM it launched on this thread (any of the
 * vdmq_gemm_* / vdmq_linear_* entry points): which kernel, its output tile, the
 * shape of the groups of tiles ("super-tiles") an XCD works on together, whether
 * every XCD walks one contiguous run of them, and the grid.  No counterpart in
 * the reference (one kernel, one tile shape, vdm_w4a4_kernel.cu:819); for tests
 * and tuning: the choice never changes a result bit.  Returns VDMQ_EINVAL when
 * nothing was launched yet. */
#define VDMQ_KERNEL_GEMM_W4A4 1           /* int8 matrix path */
#define VDMQ_KERNEL_GEMM_BF6 2            /* bf6 matrix path, one workgroup per tile (256 x 256, or 128 x 128 for small problems) */
#define VDMQ_KERNEL_GEMM_BF6_PERSISTENT 3 /* bf6 matrix path, one workgroup per CU walking tiles */
typedef struct vdmq_gemm_launch_info {
    int kernel;                 /* VDMQ_KERNEL_* */
    int tile_m, tile_n;         /* output tile of one workgroup: token rows x channels */
    int group_m, group_n;       /* super-tile, in tiles (the bf6 kernels may regroup the tile rows and columns left over at the edges) */
    int contiguous_runs;        /* 1: each XCD walks one contiguous run of super-tiles, K direction alternating */
    int64_t workgroups;         /* grid size */
} vdmq_gemm_launch_info;
int vdmq_last_gemm_launch(vdmq_gemm_launch_info *info);

/* Bytes of caller workspace vdmq_linear_w4a4 needs for an [M, K] input. */
int64_t vdmq_workspace_bytes(int64_t M, int64_t K);

/* Quantize + GEMM: linear_dynamic / linear_dynamic_bias
 * (vdm_w4a4_kernel.cu:765-838).  `workspace` holds the native qact and the
 * token scales; it replaces the reference's per-call torch::empty scratch
 * (:796-798). */
int vdmq_linear_w4a4(const void *x, int64_t M, int64_t K, int64_t ldx, float clip, const void *wq, const void *wscale,
                     const void *bias, void *out, int out_dtype, int64_t N, int64_t ldo, void *workspace,
                     int64_t workspace_bytes, vdmq_stream_t stream);

/* vdmq_linear_w4a4 with an activation fused into the quantizer (see
 * vdmq_quantize_act_ex): out = linear(act(x)). */
int vdmq_linear_w4a4_ex(const void *x, int64_t M, int64_t K, int64_t ldx, float clip, int act, const void *wq, const void *wscale,
                        const void *bias, void *out, int out_dtype, int64_t N, int64_t ldo, void *workspace,
                        int64_t workspace_bytes, vdmq_stream_t stream);

/* vdmq_linear_w4a4 with the LayerNorm (+ modulation) fused into the quantizer
 * (see vdmq_quantize_act_ln): out = linear(h). */
int vdmq_linear_ln_w4a4(const void *x, int64_t M, int64_t K, int64_t ldx, float eps, int ln_mode, const void *a, const void *b,
                        int64_t ldv, int64_t rows_per_vec, float clip, const void *wq, const void *wscale, const void *bias, void *out,
                        int out_dtype, int64_t N, int64_t ldo, void *workspace, int64_t workspace_bytes, vdmq_stream_t stream);

/* vdmq_linear_w4a4 for callers that cannot allocate device memory (code under
 * HIP graph capture, tight serving loops, harnesses that forbid hipMalloc): no
 * counterpart in the reference, whose entry points allocate their scratch with
 * torch::empty on every call.  The workspace is a buffer of
 * VDMQ_NOALLOC_SCRATCH_BYTES built into the library's device code (every GPU the
 * library is used on holds one copy until the process ends); the call allocates
 * and frees nothing.  Inputs with vdmq_workspace_bytes(M, K) beyond that size
 * are refused with VDMQ_ENOSPACE before anything is launched.  All calls on one
 * GPU share that buffer: calls that may overlap there (different streams, or
 * threads) race; calls on one stream are ordered and safe.  The first call on a
 * device looks the buffer's address up (and, like every first launch of a GEMM
 * kernel, sets its LDS size attribute): make it before a graph capture starts. */
#define VDMQ_NOALLOC_SCRATCH_BYTES (64 << 20)
int vdmq_linear_w4a4_noalloc(const void *x, int64_t M, int64_t K, int64_t ldx, float clip, const void *wq, const void *wscale,
                             const void *bias, void *out, int out_dtype, int64_t N, int64_t ldo, vdmq_stream_t stream);

/* ---- bf6 matrix path (optional; no counterpart in the reference).
 * gfx950 multiplies 6-bit floats (E3M2) at twice its int8 rate, E3M2 holds every
 * int4 value exactly -- the blocks hold q as the float q / 16, whose code is
 * sign << 5 | |q| -- and fp32 accumulation of their products is exact for
 * K <= 65536, so the same GEMM can run on v_mfma_f32_32x32x64_f8f6f4 with
 * bit-identical results.  Operands are "bf6 blocks": per row and 32 consecutive
 * k one 192-bit string of six-bit codes, stored by panels of 8 rows (a panel holds
 * its 64-deep k-blocks one after the other, 384 bytes each: [k half 0: 8 rows x
 * 16 B][half 1: 8 x 16 B][half 0: 8 x 8 B][half 1: 8 x 8 B]), rows padded to 32
 * and K to 128 with zeros (vdmq_bf6_bytes gives the size).  vdmq_native_to_bf6 converts a native int4
 * buffer (weights once per module; activations per call unless the quantizer
 * writes blocks itself); vdmq_gemm_w4a4_bf6 is vdmq_gemm_w4a4 on such operands
 * (fp16 or bf16 output), vdmq_gemm_w4a4_bf6_acc the int32 accumulator view.
 * vdmq_quantize_act_bf6 / vdmq_quantize_act_ln_bf6 are vdmq_quantize_act_ex /
 * vdmq_quantize_act_ln writing bf6 blocks (xblocks, vdmq_bf6_bytes(M, K) bytes)
 * instead of native rows: same scales, same integers; K <= 16384.
 * bf6 blocks are NOT a persistent or cross-build format: their codes changed once already (VDMQ_VERSION 1 held the
 * integers themselves, 2 holds q / 16, and the GEMM's epilogue carries the matching factor), so blocks made by another
 * build give results off by a power of two without any error.  They must come from this build's vdmq_quantize_act*_bf6
 * / vdmq_native_to_bf6 / vdmq_weight_v1_to_bf6; what is stored on disk is the v1 layout. */
int64_t vdmq_bf6_bytes(int64_t rows, int64_t K);
/* 1 when the bf6 path is the faster one for a linear of this size (quantizer + GEMM, measured on MI355X), 0
 * otherwise.  Its GEMM has 256 x 256 tiles for large problems and 128 x 128 ones for small ones and is the faster
 * GEMM on every shape measured; what decides is the quantizer, which is slower than the int4 one on short rows: the
 * path pays from K = 1280 on, whatever M and N.  A host that keeps both weight forms asks this per call; the results
 * are the same bits either way.  No counterpart in the reference (it has one matrix path). */
int vdmq_bf6_pays(int64_t M, int64_t N, int64_t K);
int vdmq_quantize_act_bf6(const void *x, int64_t M, int64_t K, int64_t ldx, float clip, int act, void *xblocks, void *scale_h,
                          vdmq_stream_t stream);
int vdmq_quantize_act_ln_bf6(const void *x, int64_t M, int64_t K, int64_t ldx, float eps, int ln_mode, const void *a, const void *b,
                             int64_t ldv, int64_t rows_per_vec, float clip, void *xblocks, void *scale_h, vdmq_stream_t stream);
/* vdmq_linear_w4a4_ex on the bf6 path: quantizer writing blocks + bf6 GEMM; wblocks = vdmq_native_to_bf6 of the
 * native weights; workspace of vdmq_workspace_bytes_bf6(M, K) bytes. */
int64_t vdmq_workspace_bytes_bf6(int64_t M, int64_t K);
int vdmq_linear_w4a4_bf6(const void *x, int64_t M, int64_t K, int64_t ldx, float clip, int act, const void *wblocks, const void *wscale,
                         const void *bias, void *out, int out_dtype, int64_t N, int64_t ldo, void *workspace, int64_t workspace_bytes,
                         vdmq_stream_t stream);
int vdmq_native_to_bf6(const void *native, int64_t rows, int64_t K, void *blocks, vdmq_stream_t stream);
/* A checkpoint's v1 weight buffer (u8 [N, K/2], weight_quantize_per_channel_kernel's order, vdm_w4a4_kernel.cu:518-551)
 * straight to bf6 blocks: the one relayout a module needs when the bf6 path serves it, made once at load.
 * Same bytes as vdmq_weight_v1_to_native followed by vdmq_native_to_bf6.  N % 128 == 0, K % 64 == 0. */
int vdmq_weight_v1_to_bf6(const void *qweight_v1, void *wblocks, int64_t N, int64_t K, vdmq_stream_t stream);
/* The inverse: bf6 weight blocks of this build back to the checkpoint's v1 buffer, byte for byte what vdmq_weight_v1_to_bf6
 * was given.  A loader that keeps only the blocks resident (3/4 byte per weight instead of 1/2 + 3/4) rebuilds the
 * state-dict tensor with it when one is asked for.  No counterpart in the reference (its kernel reads the v1 buffer). */
int vdmq_bf6_to_weight_v1(const void *wblocks, void *qweight_v1, int64_t N, int64_t K, vdmq_stream_t stream);
/* out_dtype VDMQ_OUT_F16 or VDMQ_OUT_BF16, with vdmq_gemm_w4a4's arithmetic for either */
int vdmq_gemm_w4a4_bf6(const void *xblocks, const void *ascale, const void *wblocks, const void *wscale, const void *bias, void *out,
                       int out_dtype, int64_t M, int64_t N, int64_t K, int64_t ldo, vdmq_stream_t stream);
int vdmq_gemm_w4a4_bf6_ex(const void *xblocks, const void *ascale, const void *wblocks, const void *wscale, const void *bias,
                          const void *gate, int64_t ldg, int64_t rows_per_gate, const void *residual, int64_t ldr, void *out, int out_dtype,
                          int64_t M, int64_t N, int64_t K, int64_t ldo, vdmq_stream_t stream); /* with vdmq_gemm_w4a4_ex's tail (fp16 only) */
int vdmq_gemm_w4a4_bf6_split(const void *xblocks, const void *ascale, const void *wblocks, const void *wscale, const void *bias, void *out,
                             int64_t M, int64_t N, int64_t K, int64_t ldo, int64_t split_cols, int64_t part_stride,
                             vdmq_stream_t stream); /* vdmq_gemm_w4a4_split on bf6 operands */
int vdmq_gemm_w4a4_bf6_acc(const void *xblocks, const void *wblocks, int32_t *acc, int64_t M, int64_t N, int64_t K,
                           vdmq_stream_t stream);

/* One-time relayouts between the checkpoint's v1 buffers and native ones.
 * v1 weight layout: weight_quantize_per_channel_kernel + pack_wscales
 * (vdm_w4a4_kernel.cu:518-551, :286-294).  N % 128 == 0, K % 64 == 0. */
int vdmq_weight_v1_to_native(const void *qweight_v1, void *wq_native, int64_t N, int64_t K, vdmq_stream_t stream);
int vdmq_weight_native_to_v1(const void *wq_native, void *qweight_v1, int64_t N, int64_t K, vdmq_stream_t stream);
/* packed scales fp16 [N, K/64] -> plain fp16 [N] (k-group 0, as the reference
 * GEMM reads them, :661-663) and back (repeated per k-group, :548-550). */
int vdmq_wscale_v1_to_plain(const void *packed_v1, void *plain, int64_t N, int64_t K, vdmq_stream_t stream);
int vdmq_wscale_plain_to_v1(const void *plain, void *packed_v1, int64_t N, int64_t K, vdmq_stream_t stream);

/* Activation buffers in the v1 layout, for the split entry points
 * quantize_activation_per_token / linear_prequantized
 * (vdm_w4a4_kernel.cu:840-918).  PM = ceil(M, 256); rows M..PM-1 of the v1
 * buffers are zero with scale 1 (:357-378).
 *   native_to_v1: qact u8 [M, Kp/2], scale fp16 [M] -> qact_v1 u8 [PM, K/2],
 *                 ascales_v1 fp16 [PM, K/64]
 *   v1_to_native: the inverse, for all PM rows (M % 256 == 0 required, :896). */
int vdmq_act_native_to_v1(const void *qact, const void *scale_h, int64_t M, int64_t K, void *qact_v1, void *ascales_v1,
                          vdmq_stream_t stream);
int vdmq_act_v1_to_native(const void *qact_v1, const void *ascales_v1, int64_t M, int64_t K, void *qact, void *scale_h,
                          vdmq_stream_t stream);

/* Per-row scale of an fp16 matrix with clip 1: the token_scale_kernel launch
 * of quantize_weight_per_channel (vdm_w4a4_kernel.cu:747-751). */
int vdmq_row_scale(const void *w, int64_t rows, int64_t K, float clip, void *scale_h, vdmq_stream_t stream);

/* Quantize fp16 weights [N, K] (contiguous) with caller-provided per-channel
 * fp16 scales into a native buffer: q = sat_s4(rni(float(w) * (1 / float(s))))
 * -- the arithmetic of pack_weight_with_scale / quantize_warp_static_scale
 * (vdm_w4a4_kernel.cu:697-728, :296-338).  The v1 buffers that function
 * returns are then vdmq_weight_native_to_v1 + vdmq_wscale_plain_to_v1. */
int vdmq_quantize_weight_native(const void *w, const void *scale_h, void *wq_native, int64_t N, int64_t K, vdmq_stream_t stream);

/* Plain device-to-device copy kernel with 128-bit accesses (bytes % 16 == 0).
 * No counterpart in the reference: a kernel of exactly known HBM traffic
 * (bytes read + bytes written), run next to the hot-path kernels when hardware
 * traffic counters are collected so that their readings can be scaled. */
int vdmq_copy_u128(const void *src, void *dst, int64_t bytes, vdmq_stream_t stream);

/* Streaming probe with a given mix of reads and writes (no counterpart in the reference): `threads` threads (a
 * multiple of 64) each load `reads` 16-byte vectors and store `writes` vectors -- a wave reads `reads` consecutive
 * kilobytes of src and writes `writes` consecutive kilobytes of dst, as a quantizer wave reads a row and writes a
 * shorter one -- with non-temporal accesses as the quantizers use, and do nothing else.  Mixes built in: 8 : 3 (the 2 bytes read per
 * 3/4 byte written of the A4 quantizer that writes 6-bit blocks), 4 : 1 (int4 rows), 1 : 1 (a copy), 4 : 0 (reads only;
 * the loaded values are combined but never stored, dst may be any valid pointer).  src holds threads * reads * 16
 * bytes, dst threads * writes * 16.  What it sustains is the memory system's ceiling for a kernel of that mix, which
 * the quantizers' rates are read against; timed by the caller. */
int vdmq_stream_probe(const void *src, void *dst, int64_t threads, int reads, int writes, vdmq_stream_t stream);

/* Matrix-pipe ceiling probe (no counterpart in the reference): the MFMA instruction of the int8 path
 * (VDMQ_PROBE_INT8: v_mfma_i32_32x32x32_i8) or of the bf6 path (VDMQ_PROBE_BF6: v_mfma_f32_32x32x64_f8f6f4 on
 * E3M2 operands) issued back to back -- 16 per loop iteration and wave onto 8 accumulator tiles, the GEMM kernels'
 * wave tile -- by `workgroups` workgroups of eight waves, with no memory or LDS access in the loop.  `operands`
 * holds the register contents: vdmq_mfma_probe_operand_bytes() bytes, [wave 0..7][operand 0..11][lane 0..63] x 32
 * bytes (int8 reads the first 16 of each, bf6 the first 24; operands 0-1 and 6-7 are the weight side, 2-5 and 8-11
 * the token side of the two operand sets).  `out` receives workgroups * 512 ints (a checksum that keeps the loop
 * alive); *ops the operations one launch performs (2 per multiply-accumulate).  Timed by the caller: what it sustains
 * on given operand data is the ceiling the GEMM kernels' rates are read against. */
#define VDMQ_PROBE_INT8 0
#define VDMQ_PROBE_BF6 1
int64_t vdmq_mfma_probe_operand_bytes(void);
int vdmq_mfma_probe(int kind, const void *operands, int64_t iters, int64_t workgroups, void *out, double *ops, vdmq_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* VDMQ_H */
