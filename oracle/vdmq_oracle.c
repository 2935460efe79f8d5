/*
 * CPU oracle for the W4A4 linear hot path.  TEST INFRASTRUCTURE ONLY.
 *
 * This file restates, in plain scalar C, the arithmetic of the reference's
 * CUDA source vdm_infer/kernels/csrc/vdm_w4a4_kernel.cu (IEEE reading: no
 * fast-math).  It is used by tests/, by the smoke check and by the CPU
 * baseline leg of the benchmark as the checker; the product never links or
 * calls it.
 *
 * Every function cites the reference lines it follows.  "v1 layout" is the
 * byte order the reference's CUDA packers emit (and packed checkpoints hold).
 *
 * Build: gcc -O2 -ffp-contract=off -shared -fPIC (see oracle/Makefile).
 */
#include <math.h>
#include <stdint.h>
#include <string.h>

#define BLOCK_M 256 /* vdm_w4a4_kernel.cu:15 */
#define BLOCK_N 128 /* vdm_w4a4_kernel.cu:16 */
#define WARP_K 64   /* vdm_w4a4_kernel.cu:24 */

/* ------------------------------------------------------------------ fp16 */

/* IEEE binary16 -> binary32, exact (what __half2float does). */
float vdmq_oracle_h2f(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1Fu;
    uint32_t man = h & 0x3FFu;
    uint32_t bits;
    if (exp == 0) {
        if (man == 0) {
            bits = sign;
        } else { /* subnormal: normalise */
            int e = -1;
            do {
                man <<= 1;
                ++e;
            } while (!(man & 0x400u));
            man &= 0x3FFu;
            bits = sign | ((uint32_t)(127 - 15 - e) << 23) | (man << 13);
        }
    } else if (exp == 31) {
        bits = sign | 0x7F800000u | (man << 13);
    } else {
        bits = sign | ((exp + 127 - 15) << 23) | (man << 13);
    }
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

/* binary64 -> binary16 with round-to-nearest-even, one rounding.
 * A float argument promoted to double is exact, so this is also
 * __float2half_rn (vdm_w4a4_kernel.cu:111, :479). */
uint16_t vdmq_oracle_d2h(double d) {
    uint64_t b;
    memcpy(&b, &d, 8);
    uint16_t sign = (uint16_t)((b >> 48) & 0x8000u);
    int exp = (int)((b >> 52) & 0x7FF);
    uint64_t man = b & 0xFFFFFFFFFFFFFull;
    if (exp == 0x7FF) { /* inf / nan */
        if (man == 0) return sign | 0x7C00u;
        uint16_t payload = (uint16_t)(man >> 42);
        return sign | 0x7C00u | 0x200u | payload; /* quiet */
    }
    if (exp == 0) return sign; /* double subnormals are far below half range */
    int e = exp - 1023; /* unbiased */
    uint64_t sig = man | (1ull << 52); /* 53-bit significand, value = sig * 2^(e-52) */
    /* half: normal range e in [-14, 15]; subnormal grid is 2^-24 */
    int shift; /* number of low bits of sig to drop */
    if (e >= -14) {
        shift = 42; /* keep 11 bits */
    } else {
        shift = 42 + (-14 - e); /* subnormal: fewer bits */
    }
    if (shift > 63) return sign; /* below half of the smallest subnormal */
    uint64_t kept = sig >> shift;
    uint64_t rem = sig & ((1ull << shift) - 1);
    uint64_t half = 1ull << (shift - 1);
    if (rem > half || (rem == half && (kept & 1))) kept += 1;
    uint32_t out;
    if (e >= -14) {
        /* kept in [2^10, 2^11]; 2^11 means carry into the exponent */
        int he = e + 15;
        if (kept == (1u << 11)) {
            kept >>= 1;
            he += 1;
        }
        if (he >= 31) return sign | 0x7C00u; /* overflow -> inf */
        out = ((uint32_t)he << 10) | (uint32_t)(kept & 0x3FFu);
    } else {
        /* subnormal; kept may reach 2^10 which is the smallest normal: the bit
         * pattern is then exactly right (exp field 1, mantissa 0). */
        out = (uint32_t)kept;
    }
    return sign | (uint16_t)out;
}

uint16_t vdmq_oracle_f2h(float f) { return vdmq_oracle_d2h((double)f); }

/* ------------------------------------------------------- quantizer (A1-A3) */

/* cvt.rni.s32.f32 followed by cvt.pack.sat.s4 (vdm_w4a4_kernel.cu:95-102):
 * round to nearest even integer, NaN -> 0, saturate to [-8, 7]. */
static int sat_s4_rni(float v) {
    if (v != v) return 0;
    if (v >= 7.0f) return 7; /* covers +inf and the int32 saturation */
    if (v <= -8.0f) return -8;
    float r = nearbyintf(v); /* default rounding mode: nearest even */
    return (int)r;
}

/* token_scale_kernel (vdm_w4a4_kernel.cu:459-481): per-row absmax in fp32 with
 * fmaxf (a NaN operand is ignored), scale = max > 0 ? (max / 7) * clip : 1,
 * stored as fp16 (RN).  Used for activations (clip = clip_ratio) and, in
 * quantize_weight_per_channel, for weights (clip = 1, :747-751). */
void vdmq_oracle_row_scale(const uint16_t *x, int64_t rows, int64_t K, float clip, uint16_t *scale_h) {
    for (int64_t m = 0; m < rows; ++m) {
        float mx = 0.0f;
        for (int64_t k = 0; k < K; ++k) {
            float a = fabsf(vdmq_oracle_h2f(x[m * K + k]));
            if (a == a) mx = (mx > a) ? mx : a; /* fmaxf: NaN operand ignored */
        }
        float s = mx > 0.0f ? (mx / 7.0f) * clip : 1.0f;
        scale_h[m] = vdmq_oracle_f2h(s);
    }
}

/* quantize_warp_static_scale[_guarded] (vdm_w4a4_kernel.cu:296-393), logical
 * domain: rscale = 1.0f / float(scale_h); q = sat_s4(rni(float(x) * rscale)).
 * Output one int8 per element, row-major. */
void vdmq_oracle_quantize_rows(const uint16_t *x, const uint16_t *scale_h, int64_t rows, int64_t K, int8_t *q) {
    for (int64_t m = 0; m < rows; ++m) {
        float rscale = 1.0f / vdmq_oracle_h2f(scale_h[m]);
        for (int64_t k = 0; k < K; ++k) {
            float v = vdmq_oracle_h2f(x[m * K + k]) * rscale;
            q[m * K + k] = (int8_t)sat_s4_rni(v);
        }
    }
}

/* ------------------------------------------------------------- v1 layouts */

static int64_t ceil_to(int64_t v, int64_t a) { return (v + a - 1) / a * a; }

/* Byte offset and nibble of activation element (m, k) in the v1 `qact`
 * buffer [paddedM, K/2]: act_quantize_per_token_kernel writes uint4 index
 * (((bm*KG + bk)*8 + warp)*2 + tile)*32 + lane (vdm_w4a4_kernel.cu:511) whose
 * four words are the ldmatrix.x4 result (mat[g][t], mat[g+8][t], mat[g][t+4],
 * mat[g+8][t+4]) (:334-336) of the row-major u32[16][8] tile (:313-331), and
 * element e of 8 sits in nibble e of its word (:326-329). */
int64_t vdmq_oracle_act_v1_offset(int64_t m, int64_t k, int64_t K, int *high_nibble) {
    int64_t KG = K / WARP_K;
    int64_t bm = m / BLOCK_M, warp = (m % BLOCK_M) / 32, tile = (m % 32) / 16, r = m % 16;
    int64_t g = r % 8, hi_m = r / 8;
    int64_t bk = k / WARP_K, kk = k % WARP_K, c = kk / 8, khalf = c / 4, t = c % 4;
    int64_t lane = 4 * g + t, comp = 2 * khalf + hi_m;
    *high_nibble = (int)(kk & 1);
    return (((((bm * KG + bk) * 8 + warp) * 2 + tile) * 32 + lane) * 16) + 4 * comp + (kk % 8) / 2;
}

/* Weight element (n, k) in the v1 `vdm_weight_packed` buffer [N, K/2]:
 * weight_quantize_per_channel_kernel writes uint4 index
 * ((bn*KG + bk)*8 + tile)*32 + lane (vdm_w4a4_kernel.cu:545) after swapping
 * the two middle words (:542-544), so the word order is
 * (mat[g][t], mat[g][t+4], mat[g+8][t], mat[g+8][t+4]). */
int64_t vdmq_oracle_wgt_v1_offset(int64_t n, int64_t k, int64_t K, int *high_nibble) {
    int64_t KG = K / WARP_K;
    int64_t bn = n / BLOCK_N, tile = (n % BLOCK_N) / 16, r = n % 16;
    int64_t g = r % 8, hi_n = r / 8;
    int64_t bk = k / WARP_K, kk = k % WARP_K, c = kk / 8, khalf = c / 4, t = c % 4;
    int64_t lane = 4 * g + t, comp = 2 * hi_n + khalf;
    *high_nibble = (int)(kk & 1);
    return ((((bn * KG + bk) * 8 + tile) * 32 + lane) * 16) + 4 * comp + (kk % 8) / 2;
}

/* fp16 index of (row m, k-group bk) in the v1 `ascales` buffer [paddedM, K/64]:
 * pack_ascales (vdm_w4a4_kernel.cu:276-284) written at
 * ((bm*KG + bk)*8 + warp)*16 half2 (:514-515). */
int64_t vdmq_oracle_ascale_v1_index(int64_t m, int64_t bk, int64_t K) {
    int64_t KG = K / WARP_K;
    int64_t bm = m / BLOCK_M, warp = (m % BLOCK_M) / 32, i = (m % 32) / 16, r = m % 16;
    return ((((bm * KG + bk) * 8 + warp) * 16 + 8 * i + r % 8) * 2) + r / 8;
}

/* fp16 index of (channel n, k-group bk) in `vdm_weight_scale_packed` [N, K/64]:
 * pack_wscales (vdm_w4a4_kernel.cu:286-294) written at (bn*KG + bk)*32 packs of
 * four halves (:550). */
int64_t vdmq_oracle_wscale_v1_index(int64_t n, int64_t bk, int64_t K) {
    int64_t KG = K / WARP_K;
    int64_t bn = n / BLOCK_N, j = (n % BLOCK_N) / 16, r = n % 16;
    return (((bn * KG + bk) * 32 + 4 * j + (r % 8) / 2) * 4) + 2 * (r / 8) + r % 2;
}

static void put_nibble(uint8_t *buf, int64_t off, int hi, int q) {
    uint8_t v = (uint8_t)(q & 0xF);
    if (hi)
        buf[off] = (uint8_t)((buf[off] & 0x0F) | (v << 4));
    else
        buf[off] = (uint8_t)((buf[off] & 0xF0) | v);
}

static int get_nibble(const uint8_t *buf, int64_t off, int hi) {
    int v = hi ? (buf[off] >> 4) : (buf[off] & 0xF);
    return v >= 8 ? v - 16 : v; /* two's complement int4 */
}

/* Activations q[M,K] (int8 holding int4) -> v1 qact [ceil(M,256), K/2]; rows
 * >= M are zero (vdm_w4a4_kernel.cu:357-364). */
void vdmq_oracle_pack_act_v1(const int8_t *q, int64_t M, int64_t K, uint8_t *qact) {
    int64_t PM = ceil_to(M, BLOCK_M);
    memset(qact, 0, (size_t)(PM * K / 2));
    for (int64_t m = 0; m < M; ++m)
        for (int64_t k = 0; k < K; ++k) {
            int hi;
            int64_t off = vdmq_oracle_act_v1_offset(m, k, K, &hi);
            put_nibble(qact, off, hi, q[m * K + k]);
        }
}

void vdmq_oracle_unpack_act_v1(const uint8_t *qact, int64_t M, int64_t K, int8_t *q) {
    for (int64_t m = 0; m < M; ++m)
        for (int64_t k = 0; k < K; ++k) {
            int hi;
            int64_t off = vdmq_oracle_act_v1_offset(m, k, K, &hi);
            q[m * K + k] = (int8_t)get_nibble(qact, off, hi);
        }
}

/* v1 ascales [ceil(M,256), K/64]: the row scale repeated for every k-group;
 * padded rows carry 1.0 (vdm_w4a4_kernel.cu:373-378). */
void vdmq_oracle_pack_ascales_v1(const uint16_t *scale_h, int64_t M, int64_t K, uint16_t *ascales) {
    int64_t PM = ceil_to(M, BLOCK_M), KG = K / WARP_K;
    for (int64_t m = 0; m < PM; ++m)
        for (int64_t bk = 0; bk < KG; ++bk)
            ascales[vdmq_oracle_ascale_v1_index(m, bk, K)] = m < M ? scale_h[m] : (uint16_t)0x3C00u;
}

void vdmq_oracle_pack_wgt_v1(const int8_t *q, int64_t N, int64_t K, uint8_t *qweight) {
    memset(qweight, 0, (size_t)(N * K / 2));
    for (int64_t n = 0; n < N; ++n)
        for (int64_t k = 0; k < K; ++k) {
            int hi;
            int64_t off = vdmq_oracle_wgt_v1_offset(n, k, K, &hi);
            put_nibble(qweight, off, hi, q[n * K + k]);
        }
}

void vdmq_oracle_unpack_wgt_v1(const uint8_t *qweight, int64_t N, int64_t K, int8_t *q) {
    for (int64_t n = 0; n < N; ++n)
        for (int64_t k = 0; k < K; ++k) {
            int hi;
            int64_t off = vdmq_oracle_wgt_v1_offset(n, k, K, &hi);
            q[n * K + k] = (int8_t)get_nibble(qweight, off, hi);
        }
}

void vdmq_oracle_pack_wscales_v1(const uint16_t *scale_h, int64_t N, int64_t K, uint16_t *packed) {
    int64_t KG = K / WARP_K;
    for (int64_t n = 0; n < N; ++n)
        for (int64_t bk = 0; bk < KG; ++bk) packed[vdmq_oracle_wscale_v1_index(n, bk, K)] = scale_h[n];
}

/* Channel scales as the GEMM reads them: k-group 0 only
 * (vdm_w4a4_kernel.cu:661-663). */
void vdmq_oracle_unpack_wscales_v1(const uint16_t *packed, int64_t N, int64_t K, uint16_t *scale_h) {
    for (int64_t n = 0; n < N; ++n) scale_h[n] = packed[vdmq_oracle_wscale_v1_index(n, 0, K)];
}

/* --------------------------------------------------------- GEMM + epilogue */

/* linear_w4a4_kernel main loop (vdm_w4a4_kernel.cu:671-682): exact int32
 * accumulation of qx[m,:] . qw[n,:] over the whole K. */
void vdmq_oracle_gemm_i32(const int8_t *qx, const int8_t *qw, int64_t M, int64_t N, int64_t K, int32_t *acc) {
    for (int64_t m = 0; m < M; ++m)
        for (int64_t n = 0; n < N; ++n) {
            int32_t s = 0;
            const int8_t *a = qx + m * K, *b = qw + n * K;
            for (int64_t k = 0; k < K; ++k) s += (int32_t)a[k] * (int32_t)b[k];
            acc[m * N + n] = s;
        }
}

/* finalize_int_accum + store_fpsum (vdm_w4a4_kernel.cu:243-274, 557-625):
 * s = float(as) * float(ws); h = fp16_rn(float(acc) * s); with a bias,
 * y = fp16(h + bias) as one fp16 addition (__hadd2), else y = h. */
void vdmq_oracle_epilogue(const int32_t *acc, const uint16_t *as_h, const uint16_t *ws_h, const uint16_t *bias_h, int64_t M,
                          int64_t N, uint16_t *out) {
    for (int64_t m = 0; m < M; ++m) {
        float as = vdmq_oracle_h2f(as_h[m]);
        for (int64_t n = 0; n < N; ++n) {
            float s = as * vdmq_oracle_h2f(ws_h[n]);
            float v = (float)acc[m * N + n] * s;
            uint16_t h = vdmq_oracle_f2h(v);
            if (bias_h) {
                /* the exact sum of two binary16 values fits a double */
                double y = (double)vdmq_oracle_h2f(h) + (double)vdmq_oracle_h2f(bias_h[n]);
                h = vdmq_oracle_d2h(y);
            }
            out[m * N + n] = h;
        }
    }
}

/* linear_dynamic_impl (vdm_w4a4_kernel.cu:765-830) end to end, logical
 * domain.  Scratch is caller-provided: qx [M*K] int8, as_h [M], acc [M*N]
 * (any of the three may be inspected afterwards). */
void vdmq_oracle_linear(const uint16_t *x, const int8_t *qw, const uint16_t *ws_h, const uint16_t *bias_h, float clip, int64_t M,
                        int64_t N, int64_t K, int8_t *qx, uint16_t *as_h, int32_t *acc, uint16_t *out) {
    vdmq_oracle_row_scale(x, M, K, clip, as_h);
    vdmq_oracle_quantize_rows(x, as_h, M, K, qx);
    vdmq_oracle_gemm_i32(qx, qw, M, N, K, acc);
    vdmq_oracle_epilogue(acc, as_h, ws_h, bias_h, M, N, out);
}
