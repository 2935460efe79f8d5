// extern "C" boundary of libvdmq: argument checking and dispatch only.
#include <stdarg.h>
#include <stdio.h>

#include "vdmq_internal.h"

namespace vdmq {

static thread_local char g_error[512] = "";

int fail(int code, const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
    return code;
}

static thread_local vdmq_gemm_launch_info g_last_launch = {};

void record_gemm_launch(const vdmq_gemm_launch_info &info) { g_last_launch = info; }

int check_launch(const char *what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(VDMQ_ELAUNCH, "%s: launch failed: %s", what, hipGetErrorString(e));
    return VDMQ_OK;
}

int launch_weight_relayout(const void *src, void *dst, int64_t N, int64_t K, bool to_native, hipStream_t s);
int launch_copy_u128(const void *src, void *dst, int64_t bytes, hipStream_t s);
int launch_stream_mix(const void *src, void *dst, int64_t threads, int reads, int writes, hipStream_t s);
int launch_wscale_relayout(const void *src, void *dst, int64_t N, int64_t K, bool to_plain, hipStream_t s);
int launch_act_to_v1(const void *qact, const void *scale_h, int64_t M, int64_t K, void *qact_v1, void *ascales_v1, hipStream_t s);
int launch_act_to_native(const void *qact_v1, const void *ascales_v1, int64_t M, int64_t K, void *qact, void *scale_h, hipStream_t s);

namespace {

constexpr int64_t kMaxK = 65536;      /* keeps 256 * sum(q*q) inside int32 */
constexpr int64_t kMaxLdo = 1 << 22;  /* a wave's 128 output rows stay inside the 32-bit offsets of its buffer stores */
constexpr int64_t kMaxDim = 1 << 30;  /* int indexing inside the kernels */

int check_k(int64_t K) {
    if (K <= 0 || K % VDMQ_WARP_K != 0) return fail(VDMQ_ESHAPE, "K must be a positive multiple of %d (got %lld)", VDMQ_WARP_K, (long long)K);
    if (K > kMaxK) return fail(VDMQ_ESHAPE, "K must be <= %lld (got %lld)", (long long)kMaxK, (long long)K);
    return VDMQ_OK;
}

int check_n(int64_t N) {
    if (N <= 0 || N % VDMQ_BLOCK_N != 0) return fail(VDMQ_ESHAPE, "N must be a positive multiple of %d (got %lld)", VDMQ_BLOCK_N, (long long)N);
    if (N > kMaxDim) return fail(VDMQ_ESHAPE, "shape too large for int indexing");
    return VDMQ_OK;
}

int check_m(int64_t M) {
    if (M < 0 || M > kMaxDim) return fail(VDMQ_ESHAPE, "M out of range (got %lld)", (long long)M);
    return VDMQ_OK;
}

int check_ptr(const void *p, const char *name, bool need16 = true) {
    if (p == nullptr) return fail(VDMQ_EINVAL, "%s is null", name);
    if (need16 && !aligned16(p)) return fail(VDMQ_EINVAL, "%s must be 16-byte aligned", name);
    return VDMQ_OK;
}

#define VDMQ_TRY(expr)                  \
    do {                                \
        int rc_ = (expr);               \
        if (rc_ != VDMQ_OK) return rc_; \
    } while (0)

inline hipStream_t as_stream(vdmq_stream_t s) { return static_cast<hipStream_t>(s); }

}  // namespace
}  // namespace vdmq

using namespace vdmq;

// Workspace of vdmq_linear_w4a4_noalloc: the quantized activation rows and the token scales of one call.  Every
// device the library runs on holds its own copy of the array, at its own address, until the process ends.  In host
// code the name stands for the symbol only (HIP_SYMBOL): the device address comes from hipGetSymbolAddress, once per
// device, and that pointer is what reaches the kernels.
static __device__ __align__(256) unsigned char scratch[VDMQ_NOALLOC_SCRATCH_BYTES];

namespace {

constexpr int kScratchMaxDevices = 64;
void *g_scratch_ptr[kScratchMaxDevices]; /* device address of `scratch` on device i, 0 = not asked yet */

int scratch_of_current_device(void **ptr) {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kScratchMaxDevices) {
        (void)hipGetLastError();
        return fail(VDMQ_ELAUNCH, "no current HIP device");
    }
    void *p = __atomic_load_n(&g_scratch_ptr[dev], __ATOMIC_ACQUIRE);
    if (p == nullptr) {
        const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || p == nullptr) {
            (void)hipGetLastError();
            return fail(VDMQ_ELAUNCH, "hipGetSymbolAddress(scratch) on device %d: %s", dev, hipGetErrorString(e));
        }
        __atomic_store_n(&g_scratch_ptr[dev], p, __ATOMIC_RELEASE); /* racing first calls store the same address */
    }
    *ptr = p;
    return VDMQ_OK;
}

}  // namespace

extern "C" {

int vdmq_version(void) { return VDMQ_VERSION; }
const char *vdmq_arch(void) { return "gfx950"; }
const char *vdmq_last_error(void) { return g_error; }
int64_t vdmq_k_padded(int64_t K) { return k_padded(K); }

static int quantize_act_checked(const void *x, int64_t M, int64_t K, int64_t ldx, float clip, int act, int fmt, void *qact,
                                void *scale_h, vdmq_stream_t stream) {
    VDMQ_TRY(check_k(K));
    VDMQ_TRY(check_m(M));
    if (act != VDMQ_ACT_NONE && act != VDMQ_ACT_GELU_TANH) return fail(VDMQ_EINVAL, "unknown activation %d", act);
    if (M == 0) return VDMQ_OK;
    VDMQ_TRY(check_ptr(x, "x"));
    VDMQ_TRY(check_ptr(qact, "qact"));
    VDMQ_TRY(check_ptr(scale_h, "scale_h", false));
    if (ldx < K || ldx % 8 != 0) return fail(VDMQ_ESHAPE, "ldx must be >= K and a multiple of 8 (got %lld)", (long long)ldx);
    return launch_quantize_act(static_cast<const __half *>(x), M, K, ldx, clip, act, fmt, static_cast<uint8_t *>(qact),
                               static_cast<__half *>(scale_h), as_stream(stream));
}

int vdmq_quantize_act_ex(const void *x, int64_t M, int64_t K, int64_t ldx, float clip, int act, void *qact, void *scale_h,
                         vdmq_stream_t stream) {
    return quantize_act_checked(x, M, K, ldx, clip, act, 0, qact, scale_h, stream);
}

int vdmq_quantize_act_bf6(const void *x, int64_t M, int64_t K, int64_t ldx, float clip, int act, void *xblocks, void *scale_h,
                          vdmq_stream_t stream) {
    return quantize_act_checked(x, M, K, ldx, clip, act, 1, xblocks, scale_h, stream);
}

int vdmq_quantize_act(const void *x, int64_t M, int64_t K, int64_t ldx, float clip, void *qact, void *scale_h, vdmq_stream_t stream) {
    return vdmq_quantize_act_ex(x, M, K, ldx, clip, VDMQ_ACT_NONE, qact, scale_h, stream);
}

int vdmq_gelu_tanh_f16(const void *x, void *y, int64_t n, vdmq_stream_t stream) {
    if (n < 0 || n % 2 != 0) return fail(VDMQ_ESHAPE, "n must be a non-negative even count (got %lld)", (long long)n);
    if (n == 0) return VDMQ_OK;
    VDMQ_TRY(check_ptr(x, "x", false));
    VDMQ_TRY(check_ptr(y, "y", false));
    if ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(y)) & 3u) return fail(VDMQ_EINVAL, "x and y must be 4-byte aligned");
    return launch_gelu_tanh(static_cast<const __half *>(x), static_cast<__half *>(y), n, as_stream(stream));
}

static int ln_checked(const void *x, int64_t M, int64_t K, int64_t ldx, int ln_mode, const void *a, const void *b, int64_t ldv,
                      int64_t &rows_per_vec) {
    VDMQ_TRY(check_k(K));
    VDMQ_TRY(check_m(M));
    if (K > 16384) return fail(VDMQ_ESHAPE, "the fused LayerNorm needs K <= 16384 (got %lld)", (long long)K);
    if (ln_mode != VDMQ_LN_MODULATE && ln_mode != VDMQ_LN_AFFINE) return fail(VDMQ_EINVAL, "unknown ln_mode %d", ln_mode);
    if (rows_per_vec <= 0) return fail(VDMQ_ESHAPE, "rows_per_vec must be positive (got %lld)", (long long)rows_per_vec);
    if (rows_per_vec > (int64_t(1) << 30)) rows_per_vec = int64_t(1) << 30; /* "one vector for every row": the kernels index with int */
    if (ldv < K || ldv % 8 != 0) return fail(VDMQ_ESHAPE, "ldv must be >= K and a multiple of 8 (got %lld)", (long long)ldv);
    if (ldx < K || ldx % 8 != 0) return fail(VDMQ_ESHAPE, "ldx must be >= K and a multiple of 8 (got %lld)", (long long)ldx);
    if (M == 0) return VDMQ_OK;
    VDMQ_TRY(check_ptr(x, "x"));
    VDMQ_TRY(check_ptr(a, "a"));
    VDMQ_TRY(check_ptr(b, "b"));
    return VDMQ_OK;
}

static int quantize_act_ln_checked(const void *x, int64_t M, int64_t K, int64_t ldx, float eps, int ln_mode, const void *a, const void *b,
                                   int64_t ldv, int64_t rows_per_vec, float clip, int fmt, void *qact, void *scale_h,
                                   vdmq_stream_t stream) {
    VDMQ_TRY(ln_checked(x, M, K, ldx, ln_mode, a, b, ldv, rows_per_vec));
    if (M == 0) return VDMQ_OK;
    VDMQ_TRY(check_ptr(qact, "qact"));
    VDMQ_TRY(check_ptr(scale_h, "scale_h", false));
    return launch_ln_quantize(static_cast<const __half *>(x), M, K, ldx, eps, ln_mode, static_cast<const __half *>(a),
                              static_cast<const __half *>(b), ldv, rows_per_vec, clip, fmt, static_cast<uint8_t *>(qact),
                              static_cast<__half *>(scale_h), nullptr, 0, as_stream(stream));
}

int vdmq_quantize_act_ln(const void *x, int64_t M, int64_t K, int64_t ldx, float eps, int ln_mode, const void *a, const void *b,
                         int64_t ldv, int64_t rows_per_vec, float clip, void *qact, void *scale_h, vdmq_stream_t stream) {
    return quantize_act_ln_checked(x, M, K, ldx, eps, ln_mode, a, b, ldv, rows_per_vec, clip, 0, qact, scale_h, stream);
}

int vdmq_quantize_act_ln_bf6(const void *x, int64_t M, int64_t K, int64_t ldx, float eps, int ln_mode, const void *a, const void *b,
                             int64_t ldv, int64_t rows_per_vec, float clip, void *xblocks, void *scale_h, vdmq_stream_t stream) {
    return quantize_act_ln_checked(x, M, K, ldx, eps, ln_mode, a, b, ldv, rows_per_vec, clip, 1, xblocks, scale_h, stream);
}

int vdmq_ln_f16(const void *x, int64_t M, int64_t K, int64_t ldx, float eps, int ln_mode, const void *a, const void *b, int64_t ldv,
                int64_t rows_per_vec, void *h, int64_t ldh, vdmq_stream_t stream) {
    VDMQ_TRY(ln_checked(x, M, K, ldx, ln_mode, a, b, ldv, rows_per_vec));
    if (M == 0) return VDMQ_OK;
    VDMQ_TRY(check_ptr(h, "h"));
    if (ldh < K || ldh % 8 != 0) return fail(VDMQ_ESHAPE, "ldh must be >= K and a multiple of 8 (got %lld)", (long long)ldh);
    return launch_ln_quantize(static_cast<const __half *>(x), M, K, ldx, eps, ln_mode, static_cast<const __half *>(a),
                              static_cast<const __half *>(b), ldv, rows_per_vec, 1.0f, 0, nullptr, nullptr, static_cast<__half *>(h), ldh,
                              as_stream(stream));
}

static int check_tail(const GemmTail &tail, int64_t N) {
    if (tail.gate != nullptr) {
        VDMQ_TRY(check_ptr(tail.gate, "gate"));
        if (tail.ldg < N || tail.ldg % 8 != 0) return fail(VDMQ_ESHAPE, "ldg must be >= N and a multiple of 8 (got %lld)", (long long)tail.ldg);
        if (tail.rows_per_gate <= 0) return fail(VDMQ_ESHAPE, "rows_per_gate must be positive");
    }
    if (tail.residual != nullptr) {
        VDMQ_TRY(check_ptr(tail.residual, "residual"));
        if (tail.ldr < N || tail.ldr % 8 != 0) return fail(VDMQ_ESHAPE, "ldr must be >= N and a multiple of 8 (got %lld)", (long long)tail.ldr);
    }
    return VDMQ_OK;
}

static GemmTail make_tail(const void *gate, int64_t ldg, int64_t rows_per_gate, const void *residual, int64_t ldr) {
    if (rows_per_gate > (int64_t(1) << 30)) rows_per_gate = int64_t(1) << 30; /* "one gate vector for every row" */
    GemmTail tail;
    tail.gate = static_cast<const __half *>(gate);
    tail.ldg = ldg;
    tail.rows_per_gate = static_cast<int>(rows_per_gate);
    tail.residual = static_cast<const __half *>(residual);
    tail.ldr = ldr;
    return tail;
}

// Output split of vdmq_gemm_w4a4_split: checks, and the columns a row of `out` has to hold
static int check_split(GemmTail &tail, int64_t N, int64_t split_cols, int64_t part_stride) {
    if (split_cols <= 0 || split_cols % 64 != 0 || N % split_cols != 0)
        return fail(VDMQ_ESHAPE, "split_cols must be a positive multiple of 64 that divides N (got %lld, N = %lld)", (long long)split_cols, (long long)N);
    if (part_stride < 0 || part_stride % 8 != 0) return fail(VDMQ_ESHAPE, "part_stride must be a non-negative multiple of 8 (got %lld)", (long long)part_stride);
    tail.split_cols = static_cast<int>(split_cols);
    tail.part_stride = part_stride;
    return VDMQ_OK;
}

static int gemm_checked(const void *qact, const void *ascale, const void *wq, const void *wscale, const void *bias, void *out,
                        int out_dtype, int32_t *acc, int64_t M, int64_t N, int64_t K, int64_t ldo, const GemmTail &tail,
                        vdmq_stream_t stream) {
    VDMQ_TRY(check_k(K));
    VDMQ_TRY(check_n(N));
    VDMQ_TRY(check_m(M));
    if (M == 0) return VDMQ_OK;
    VDMQ_TRY(check_ptr(qact, "qact"));
    VDMQ_TRY(check_ptr(wq, "wq"));
    if (acc == nullptr) {
        VDMQ_TRY(check_ptr(ascale, "ascale", false));
        VDMQ_TRY(check_ptr(wscale, "wscale"));
        VDMQ_TRY(check_ptr(out, "out"));
        if (bias != nullptr) VDMQ_TRY(check_ptr(bias, "bias"));
        if (out_dtype != VDMQ_OUT_F16 && out_dtype != VDMQ_OUT_BF16) return fail(VDMQ_EINVAL, "unknown out_dtype %d", out_dtype);
        if (ldo < (tail.split_cols ? tail.split_cols : N) || ldo % 8 != 0 || ldo > kMaxLdo)
            return fail(VDMQ_ESHAPE, "ldo must be >= the columns of a row, a multiple of 8 and at most %lld (got %lld)", (long long)kMaxLdo, (long long)ldo);
        if (tail.gate != nullptr || tail.residual != nullptr || tail.split_cols != 0) {
            if (out_dtype != VDMQ_OUT_F16) return fail(VDMQ_EINVAL, "gate, residual and a split output need an fp16 output");
            VDMQ_TRY(check_tail(tail, N));
        }
    } else {
        VDMQ_TRY(check_ptr(acc, "acc"));
    }
    return launch_gemm(static_cast<const uint8_t *>(qact), static_cast<const __half *>(ascale), static_cast<const uint8_t *>(wq),
                       static_cast<const __half *>(wscale), static_cast<const __half *>(bias), out, out_dtype, acc, M, N, K, ldo, tail,
                       as_stream(stream));
}

int vdmq_gemm_w4a4(const void *qact, const void *ascale, const void *wq, const void *wscale, const void *bias, void *out,
                   int out_dtype, int64_t M, int64_t N, int64_t K, int64_t ldo, vdmq_stream_t stream) {
    return gemm_checked(qact, ascale, wq, wscale, bias, out, out_dtype, nullptr, M, N, K, ldo, GemmTail{}, stream);
}

int vdmq_gemm_w4a4_ex(const void *qact, const void *ascale, const void *wq, const void *wscale, const void *bias, const void *gate,
                      int64_t ldg, int64_t rows_per_gate, const void *residual, int64_t ldr, void *out, int out_dtype, int64_t M,
                      int64_t N, int64_t K, int64_t ldo, vdmq_stream_t stream) {
    return gemm_checked(qact, ascale, wq, wscale, bias, out, out_dtype, nullptr, M, N, K, ldo, make_tail(gate, ldg, rows_per_gate, residual, ldr),
                        stream);
}

int vdmq_gemm_w4a4_split(const void *qact, const void *ascale, const void *wq, const void *wscale, const void *bias, void *out, int64_t M,
                         int64_t N, int64_t K, int64_t ldo, int64_t split_cols, int64_t part_stride, vdmq_stream_t stream) {
    GemmTail tail;
    VDMQ_TRY(check_split(tail, N, split_cols, part_stride));
    return gemm_checked(qact, ascale, wq, wscale, bias, out, VDMQ_OUT_F16, nullptr, M, N, K, ldo, tail, stream);
}

int vdmq_gemm_w4a4_acc(const void *qact, const void *wq, int32_t *acc, int64_t M, int64_t N, int64_t K, vdmq_stream_t stream) {
    if (acc == nullptr && M != 0) return fail(VDMQ_EINVAL, "acc is null");
    return gemm_checked(qact, nullptr, wq, nullptr, nullptr, nullptr, VDMQ_OUT_F16, acc, M, N, K, N, GemmTail{}, stream);
}

int vdmq_last_gemm_launch(vdmq_gemm_launch_info *info) {
    if (info == nullptr) return fail(VDMQ_EINVAL, "info is null");
    if (g_last_launch.kernel == 0) return fail(VDMQ_EINVAL, "no GEMM was launched on this thread yet");
    *info = g_last_launch;
    return VDMQ_OK;
}

int64_t vdmq_workspace_bytes(int64_t M, int64_t K) {
    if (M < 0 || K <= 0) return 0;
    const int64_t q = (M * (k_padded(K) / 2) + 255) / 256 * 256;
    return q + (M * 2 + 255) / 256 * 256;
}

int vdmq_linear_w4a4_ex(const void *x, int64_t M, int64_t K, int64_t ldx, float clip, int act, const void *wq, const void *wscale,
                        const void *bias, void *out, int out_dtype, int64_t N, int64_t ldo, void *workspace, int64_t workspace_bytes,
                        vdmq_stream_t stream) {
    VDMQ_TRY(check_k(K));
    VDMQ_TRY(check_n(N));
    VDMQ_TRY(check_m(M));
    if (M == 0) return VDMQ_OK;
    VDMQ_TRY(check_ptr(workspace, "workspace"));
    if (workspace_bytes < vdmq_workspace_bytes(M, K))
        return fail(VDMQ_ENOSPACE, "workspace has %lld bytes, %lld needed", (long long)workspace_bytes,
                    (long long)vdmq_workspace_bytes(M, K));
    uint8_t *qact = static_cast<uint8_t *>(workspace);
    void *scale = qact + (M * (k_padded(K) / 2) + 255) / 256 * 256;
    VDMQ_TRY(vdmq_quantize_act_ex(x, M, K, ldx, clip, act, qact, scale, stream));
    return vdmq_gemm_w4a4(qact, scale, wq, wscale, bias, out, out_dtype, M, N, K, ldo, stream);
}

int vdmq_linear_ln_w4a4(const void *x, int64_t M, int64_t K, int64_t ldx, float eps, int ln_mode, const void *a, const void *b,
                        int64_t ldv, int64_t rows_per_vec, float clip, const void *wq, const void *wscale, const void *bias, void *out,
                        int out_dtype, int64_t N, int64_t ldo, void *workspace, int64_t workspace_bytes, vdmq_stream_t stream) {
    VDMQ_TRY(check_k(K));
    VDMQ_TRY(check_n(N));
    VDMQ_TRY(check_m(M));
    if (M == 0) return VDMQ_OK;
    VDMQ_TRY(check_ptr(workspace, "workspace"));
    if (workspace_bytes < vdmq_workspace_bytes(M, K))
        return fail(VDMQ_ENOSPACE, "workspace has %lld bytes, %lld needed", (long long)workspace_bytes,
                    (long long)vdmq_workspace_bytes(M, K));
    uint8_t *qact = static_cast<uint8_t *>(workspace);
    void *scale = qact + (M * (k_padded(K) / 2) + 255) / 256 * 256;
    VDMQ_TRY(vdmq_quantize_act_ln(x, M, K, ldx, eps, ln_mode, a, b, ldv, rows_per_vec, clip, qact, scale, stream));
    return vdmq_gemm_w4a4(qact, scale, wq, wscale, bias, out, out_dtype, M, N, K, ldo, stream);
}

int vdmq_linear_w4a4(const void *x, int64_t M, int64_t K, int64_t ldx, float clip, const void *wq, const void *wscale,
                     const void *bias, void *out, int out_dtype, int64_t N, int64_t ldo, void *workspace, int64_t workspace_bytes,
                     vdmq_stream_t stream) {
    return vdmq_linear_w4a4_ex(x, M, K, ldx, clip, VDMQ_ACT_NONE, wq, wscale, bias, out, out_dtype, N, ldo, workspace, workspace_bytes,
                               stream);
}

int vdmq_linear_w4a4_noalloc(const void *x, int64_t M, int64_t K, int64_t ldx, float clip, const void *wq, const void *wscale,
                             const void *bias, void *out, int out_dtype, int64_t N, int64_t ldo, vdmq_stream_t stream) {
    VDMQ_TRY(check_k(K));
    VDMQ_TRY(check_n(N));
    VDMQ_TRY(check_m(M));
    const int64_t need = vdmq_workspace_bytes(M, K);
    if (need > static_cast<int64_t>(VDMQ_NOALLOC_SCRATCH_BYTES))
        return fail(VDMQ_ENOSPACE, "an [M = %lld, K = %lld] input needs %lld bytes of scratch, the built-in buffer holds %lld",
                    (long long)M, (long long)K, (long long)need, (long long)VDMQ_NOALLOC_SCRATCH_BYTES);
    if (M == 0) return VDMQ_OK;
    void *ws = nullptr;
    VDMQ_TRY(scratch_of_current_device(&ws));
    // the quantizer writes every byte the GEMM reads (all M rows with their padding, all M scales): nothing of the
    // previous call's contents is seen, nothing has to be cleared
    return vdmq_linear_w4a4_ex(x, M, K, ldx, clip, VDMQ_ACT_NONE, wq, wscale, bias, out, out_dtype, N, ldo, ws, need, stream);
}

int64_t vdmq_bf6_bytes(int64_t rows, int64_t K) {
    if (rows < 0 || K <= 0) return 0;
    return bf6_bytes(rows, K);
}

int vdmq_native_to_bf6(const void *native, int64_t rows, int64_t K, void *blocks, vdmq_stream_t stream) {
    VDMQ_TRY(check_k(K));
    VDMQ_TRY(check_m(rows));
    if (rows == 0) return VDMQ_OK;
    VDMQ_TRY(check_ptr(native, "native"));
    VDMQ_TRY(check_ptr(blocks, "blocks"));
    return launch_nibbles_to_bf6(static_cast<const uint8_t *>(native), rows, K, static_cast<uint8_t *>(blocks), as_stream(stream));
}

int vdmq_weight_v1_to_bf6(const void *qweight_v1, void *wblocks, int64_t N, int64_t K, vdmq_stream_t stream) {
    VDMQ_TRY(check_k(K));
    VDMQ_TRY(check_n(N));
    VDMQ_TRY(check_ptr(qweight_v1, "qweight_v1"));
    VDMQ_TRY(check_ptr(wblocks, "wblocks"));
    return launch_weight_v1_to_bf6(static_cast<const uint8_t *>(qweight_v1), N, K, static_cast<uint8_t *>(wblocks), as_stream(stream));
}

int vdmq_bf6_to_weight_v1(const void *wblocks, void *qweight_v1, int64_t N, int64_t K, vdmq_stream_t stream) {
    VDMQ_TRY(check_k(K));
    VDMQ_TRY(check_n(N));
    VDMQ_TRY(check_ptr(qweight_v1, "qweight_v1"));
    VDMQ_TRY(check_ptr(wblocks, "wblocks"));
    return launch_bf6_to_weight_v1(static_cast<const uint8_t *>(wblocks), N, K, static_cast<uint8_t *>(qweight_v1), as_stream(stream));
}

static int gemm_bf6_checked(const void *xblocks, const void *ascale, const void *wblocks, const void *wscale, const void *bias, void *out,
                            int out_dtype, int32_t *acc, int64_t M, int64_t N, int64_t K, int64_t ldo, const GemmTail &tail,
                            vdmq_stream_t stream) {
    VDMQ_TRY(check_k(K));
    VDMQ_TRY(check_n(N));
    VDMQ_TRY(check_m(M));
    if (M == 0) return VDMQ_OK;
    VDMQ_TRY(check_ptr(xblocks, "xblocks"));
    VDMQ_TRY(check_ptr(wblocks, "wblocks"));
    if (acc == nullptr) {
        VDMQ_TRY(check_ptr(ascale, "ascale", false));
        VDMQ_TRY(check_ptr(wscale, "wscale"));
        VDMQ_TRY(check_ptr(out, "out"));
        if (bias != nullptr) VDMQ_TRY(check_ptr(bias, "bias"));
        if (out_dtype != VDMQ_OUT_F16 && out_dtype != VDMQ_OUT_BF16) return fail(VDMQ_EINVAL, "unknown out_dtype %d", out_dtype);
        if (ldo < (tail.split_cols ? tail.split_cols : N) || ldo % 8 != 0 || ldo > kMaxLdo)
            return fail(VDMQ_ESHAPE, "ldo must be >= the columns of a row, a multiple of 8 and at most %lld (got %lld)", (long long)kMaxLdo, (long long)ldo);
        if (tail.gate != nullptr || tail.residual != nullptr || tail.split_cols != 0) {
            if (out_dtype != VDMQ_OUT_F16) return fail(VDMQ_EINVAL, "gate, residual and a split output need an fp16 output");
            VDMQ_TRY(check_tail(tail, N));
        }
    } else {
        VDMQ_TRY(check_ptr(acc, "acc"));
    }
    return launch_gemm_bf6(static_cast<const uint8_t *>(xblocks), static_cast<const __half *>(ascale), static_cast<const uint8_t *>(wblocks),
                           static_cast<const __half *>(wscale), static_cast<const __half *>(bias), out, out_dtype, acc, M, N, K, ldo, tail,
                           as_stream(stream));
}

int vdmq_gemm_w4a4_bf6(const void *xblocks, const void *ascale, const void *wblocks, const void *wscale, const void *bias, void *out,
                       int out_dtype, int64_t M, int64_t N, int64_t K, int64_t ldo, vdmq_stream_t stream) {
    return gemm_bf6_checked(xblocks, ascale, wblocks, wscale, bias, out, out_dtype, nullptr, M, N, K, ldo, GemmTail{}, stream);
}

int vdmq_gemm_w4a4_bf6_ex(const void *xblocks, const void *ascale, const void *wblocks, const void *wscale, const void *bias,
                          const void *gate, int64_t ldg, int64_t rows_per_gate, const void *residual, int64_t ldr, void *out, int out_dtype,
                          int64_t M, int64_t N, int64_t K, int64_t ldo, vdmq_stream_t stream) {
    return gemm_bf6_checked(xblocks, ascale, wblocks, wscale, bias, out, out_dtype, nullptr, M, N, K, ldo,
                            make_tail(gate, ldg, rows_per_gate, residual, ldr), stream);
}

int vdmq_gemm_w4a4_bf6_split(const void *xblocks, const void *ascale, const void *wblocks, const void *wscale, const void *bias, void *out,
                             int64_t M, int64_t N, int64_t K, int64_t ldo, int64_t split_cols, int64_t part_stride, vdmq_stream_t stream) {
    GemmTail tail;
    VDMQ_TRY(check_split(tail, N, split_cols, part_stride));
    return gemm_bf6_checked(xblocks, ascale, wblocks, wscale, bias, out, VDMQ_OUT_F16, nullptr, M, N, K, ldo, tail, stream);
}

int vdmq_gemm_w4a4_bf6_acc(const void *xblocks, const void *wblocks, int32_t *acc, int64_t M, int64_t N, int64_t K,
                           vdmq_stream_t stream) {
    if (acc == nullptr && M != 0) return fail(VDMQ_EINVAL, "acc is null");
    return gemm_bf6_checked(xblocks, nullptr, wblocks, nullptr, nullptr, nullptr, VDMQ_OUT_F16, acc, M, N, K, N, GemmTail{}, stream);
}

int vdmq_bf6_pays(int64_t M, int64_t N, int64_t K) {
    if (M <= 0 || N <= 0 || K <= 0) return 0;
    // Measured, quantizer + GEMM, int8 time / bf6 time on 180 shapes (M 1 ... 32768, N 128 ... 15360).  K >= 1536: 1.01 ...
    // 1.97 everywhere but one shape at 0.96 (512 x 5120 -> 10240 1.44, 4096 x 1536 -> 4608 1.01, 8192 x 5120 -> 10240
    // 1.42, 100 x 5120 -> 15360 1.97).  K = 1280: 1.05 ... 1.36 on 12 of 16 shapes, 0.80 ... 0.98 on four.  K = 1024: 11 : 5,
    // K = 768: 9 : 7 (0.76 ... 1.27); K <= 512: 0.73 ... 1.03 -- the quantizer that writes blocks is the slower one on short
    // rows and decides such a linear.  M and N no longer matter since the GEMM has a small-tile configuration.
    return K >= 1280 ? 1 : 0;
}

int64_t vdmq_workspace_bytes_bf6(int64_t M, int64_t K) {
    if (M < 0 || K <= 0) return 0;
    return (bf6_bytes(M, K) + 255) / 256 * 256 + (M * 2 + 255) / 256 * 256;
}

int vdmq_linear_w4a4_bf6(const void *x, int64_t M, int64_t K, int64_t ldx, float clip, int act, const void *wblocks, const void *wscale,
                         const void *bias, void *out, int out_dtype, int64_t N, int64_t ldo, void *workspace, int64_t workspace_bytes,
                         vdmq_stream_t stream) {
    VDMQ_TRY(check_k(K));
    VDMQ_TRY(check_n(N));
    VDMQ_TRY(check_m(M));
    if (M == 0) return VDMQ_OK;
    VDMQ_TRY(check_ptr(workspace, "workspace"));
    if (workspace_bytes < vdmq_workspace_bytes_bf6(M, K))
        return fail(VDMQ_ENOSPACE, "workspace has %lld bytes, %lld needed", (long long)workspace_bytes,
                    (long long)vdmq_workspace_bytes_bf6(M, K));
    uint8_t *xblocks = static_cast<uint8_t *>(workspace);
    void *scale = xblocks + (bf6_bytes(M, K) + 255) / 256 * 256;
    VDMQ_TRY(vdmq_quantize_act_bf6(x, M, K, ldx, clip, act, xblocks, scale, stream));
    return vdmq_gemm_w4a4_bf6(xblocks, scale, wblocks, wscale, bias, out, out_dtype, M, N, K, ldo, stream);
}

int vdmq_weight_v1_to_native(const void *qweight_v1, void *wq_native, int64_t N, int64_t K, vdmq_stream_t stream) {
    VDMQ_TRY(check_k(K));
    VDMQ_TRY(check_n(N));
    VDMQ_TRY(check_ptr(qweight_v1, "qweight_v1"));
    VDMQ_TRY(check_ptr(wq_native, "wq_native"));
    return launch_weight_relayout(qweight_v1, wq_native, N, K, true, as_stream(stream));
}

int vdmq_weight_native_to_v1(const void *wq_native, void *qweight_v1, int64_t N, int64_t K, vdmq_stream_t stream) {
    VDMQ_TRY(check_k(K));
    VDMQ_TRY(check_n(N));
    VDMQ_TRY(check_ptr(qweight_v1, "qweight_v1"));
    VDMQ_TRY(check_ptr(wq_native, "wq_native"));
    return launch_weight_relayout(wq_native, qweight_v1, N, K, false, as_stream(stream));
}

int vdmq_wscale_v1_to_plain(const void *packed_v1, void *plain, int64_t N, int64_t K, vdmq_stream_t stream) {
    VDMQ_TRY(check_k(K));
    VDMQ_TRY(check_n(N));
    VDMQ_TRY(check_ptr(packed_v1, "packed_v1", false));
    VDMQ_TRY(check_ptr(plain, "plain", false));
    return launch_wscale_relayout(packed_v1, plain, N, K, true, as_stream(stream));
}

int vdmq_wscale_plain_to_v1(const void *plain, void *packed_v1, int64_t N, int64_t K, vdmq_stream_t stream) {
    VDMQ_TRY(check_k(K));
    VDMQ_TRY(check_n(N));
    VDMQ_TRY(check_ptr(packed_v1, "packed_v1", false));
    VDMQ_TRY(check_ptr(plain, "plain", false));
    return launch_wscale_relayout(plain, packed_v1, N, K, false, as_stream(stream));
}

int vdmq_act_native_to_v1(const void *qact, const void *scale_h, int64_t M, int64_t K, void *qact_v1, void *ascales_v1,
                          vdmq_stream_t stream) {
    VDMQ_TRY(check_k(K));
    VDMQ_TRY(check_m(M));
    if (M == 0) return VDMQ_OK;
    VDMQ_TRY(check_ptr(qact, "qact"));
    VDMQ_TRY(check_ptr(scale_h, "scale_h", false));
    VDMQ_TRY(check_ptr(qact_v1, "qact_v1"));
    VDMQ_TRY(check_ptr(ascales_v1, "ascales_v1", false));
    return launch_act_to_v1(qact, scale_h, M, K, qact_v1, ascales_v1, as_stream(stream));
}

int vdmq_act_v1_to_native(const void *qact_v1, const void *ascales_v1, int64_t M, int64_t K, void *qact, void *scale_h,
                          vdmq_stream_t stream) {
    VDMQ_TRY(check_k(K));
    VDMQ_TRY(check_m(M));
    if (M % VDMQ_BLOCK_M != 0) return fail(VDMQ_ESHAPE, "M must be a multiple of %d (got %lld)", VDMQ_BLOCK_M, (long long)M);
    if (M == 0) return VDMQ_OK;
    VDMQ_TRY(check_ptr(qact, "qact"));
    VDMQ_TRY(check_ptr(scale_h, "scale_h", false));
    VDMQ_TRY(check_ptr(qact_v1, "qact_v1"));
    VDMQ_TRY(check_ptr(ascales_v1, "ascales_v1", false));
    return launch_act_to_native(qact_v1, ascales_v1, M, K, qact, scale_h, as_stream(stream));
}

int vdmq_row_scale(const void *w, int64_t rows, int64_t K, float clip, void *scale_h, vdmq_stream_t stream) {
    VDMQ_TRY(check_k(K));
    VDMQ_TRY(check_m(rows));
    if (rows == 0) return VDMQ_OK;
    VDMQ_TRY(check_ptr(w, "w"));
    VDMQ_TRY(check_ptr(scale_h, "scale_h", false));
    return launch_row_scale(static_cast<const __half *>(w), rows, K, clip, static_cast<__half *>(scale_h), as_stream(stream));
}

int vdmq_copy_u128(const void *src, void *dst, int64_t bytes, vdmq_stream_t stream) {
    if (bytes < 0 || bytes % 16 != 0 || bytes / 16 > (int64_t(1) << 31) * 255) return fail(VDMQ_ESHAPE, "bytes must be a non-negative multiple of 16");
    if (bytes == 0) return VDMQ_OK;
    VDMQ_TRY(check_ptr(src, "src"));
    VDMQ_TRY(check_ptr(dst, "dst"));
    return launch_copy_u128(src, dst, bytes, as_stream(stream));
}

int vdmq_stream_probe(const void *src, void *dst, int64_t threads, int reads, int writes, vdmq_stream_t stream) {
    if (threads < 0 || threads % 64 != 0 || threads > (int64_t(1) << 31) * 255)
        return fail(VDMQ_ESHAPE, "threads must be a non-negative multiple of 64 (got %lld)", (long long)threads);
    if (threads == 0) return VDMQ_OK;
    VDMQ_TRY(check_ptr(src, "src"));
    VDMQ_TRY(check_ptr(dst, "dst"));
    return launch_stream_mix(src, dst, threads, reads, writes, as_stream(stream));
}

int vdmq_quantize_weight_native(const void *w, const void *scale_h, void *wq_native, int64_t N, int64_t K, vdmq_stream_t stream) {
    VDMQ_TRY(check_k(K));
    VDMQ_TRY(check_n(N));
    VDMQ_TRY(check_ptr(w, "w"));
    VDMQ_TRY(check_ptr(scale_h, "scale_h", false));
    VDMQ_TRY(check_ptr(wq_native, "wq_native"));
    return launch_quantize_given_scale(static_cast<const __half *>(w), static_cast<const __half *>(scale_h), N, K,
                                       static_cast<uint8_t *>(wq_native), as_stream(stream));
}

int64_t vdmq_mfma_probe_operand_bytes(void) { return mfma_probe_operand_bytes(); }

int vdmq_mfma_probe(int kind, const void *operands, int64_t iters, int64_t workgroups, void *out, double *ops, vdmq_stream_t stream) {
    if (kind != VDMQ_PROBE_INT8 && kind != VDMQ_PROBE_BF6) return fail(VDMQ_EINVAL, "unknown probe kind %d", kind);
    if (iters <= 0 || iters > (1 << 30) || workgroups <= 0 || workgroups > (1 << 20))
        return fail(VDMQ_ESHAPE, "iters and workgroups must be positive (got %lld, %lld)", (long long)iters, (long long)workgroups);
    if (ops == nullptr) return fail(VDMQ_EINVAL, "ops is null");
    VDMQ_TRY(check_ptr(operands, "operands"));
    VDMQ_TRY(check_ptr(out, "out"));
    return launch_mfma_probe(kind, operands, static_cast<int>(iters), static_cast<int>(workgroups), out, ops, as_stream(stream));
}

}  // extern "C"
