// Dynamic per-token A4 quantizer for gfx950: one pass over X.
//
// One 64-lane wave owns one token row.  The row is read once with 128-bit
// loads and kept in registers; the absmax is reduced on the packed fp16 bit
// patterns (exact, order-free); the scale is rounded to fp16; every element is
// multiplied by the fp32 reciprocal of that fp16 scale, rounded half-to-even
// and saturated to [-8, 7]; eight results are packed into one 32-bit word and
// stored row-major (element e of a word in nibble e).
//
// Arithmetic contract (IEEE reading of vdm_w4a4_kernel.cu:459-481, 95-102,
// 319-329 of the reference): see quantize_word_exact below, which spells it
// out literally and serves rows that contain NaN/Inf or whose fp16 scale is
// zero/non-finite; all other rows take a shorter, bit-identical sequence.
#include "vdmq_internal.h"

namespace vdmq {
namespace {

typedef unsigned short u16x2 __attribute__((ext_vector_type(2)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ uint32_t pk_max_u16(uint32_t a, uint32_t b) {
    u16x2 r = __builtin_elementwise_max(__builtin_bit_cast(u16x2, a), __builtin_bit_cast(u16x2, b));
    return __builtin_bit_cast(uint32_t, r);
}

__device__ __forceinline__ float half_bits_to_float(uint32_t bits16) {
    return static_cast<float>(__builtin_bit_cast(_Float16, static_cast<unsigned short>(bits16)));
}

template <typename T>
__device__ __forceinline__ T wave_max(T v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        T o = __shfl_xor(v, off, 64);
        v = o > v ? o : v;
    }
    return v;
}

// fmaxf semantics of the reference's reduction: a NaN operand is ignored.
__device__ __forceinline__ float max_ignoring_nan(float acc, float a) { return (a == a && a > acc) ? a : acc; }

// cvt.rni.s32.f32 + cvt.pack.sat.s4: NaN -> 0, saturate, round half to even.
__device__ __forceinline__ uint32_t sat_s4_rni(float v) {
    if (v != v) return 0u;
    if (v >= 7.0f) return 7u;
    if (v <= -8.0f) return 8u; /* -8 as a nibble */
    return static_cast<uint32_t>(static_cast<int>(__builtin_rintf(v))) & 0xFu;
}

// Literal form: q = sat_s4(rni(float(x) * rscale)) for the two halves of `w`.
__device__ __forceinline__ uint32_t quantize_pair_exact(uint32_t w, float rscale) {
    float lo = half_bits_to_float(w & 0xFFFFu) * rscale;
    float hi = half_bits_to_float(w >> 16) * rscale;
    return sat_s4_rni(lo) | (sat_s4_rni(hi) << 4);
}

__device__ __forceinline__ uint32_t quantize_word_exact(u32x4 v, float rscale) {
    return quantize_pair_exact(v.x, rscale) | (quantize_pair_exact(v.y, rscale) << 8) |
           (quantize_pair_exact(v.z, rscale) << 16) | (quantize_pair_exact(v.w, rscale) << 24);
}

// Fast form for finite inputs and a finite non-zero scale.  t = clamp(v) is
// rounded to an integer by adding 1.5*2^23 + 8 (the fp32 adder rounds half to
// even on the unit grid there), which leaves u = rni(t) + 8 in [0, 15] in the
// low bits of the sum: bits = 0x4B400000 + u.  Eight sums are combined with
// shift-adds; the constant parts add up to 0x4B400000 * 0x11111111 (mod 2^32)
// and are removed at the end; u ^ 8 is the two's complement nibble.
constexpr float kMagic = 12582920.0f; /* 1.5 * 2^23 + 8 */
constexpr uint32_t kMagicSum = static_cast<uint32_t>(0x4B400000ull * 0x11111111ull);

__device__ __forceinline__ uint32_t quantize_word_fast(u32x4 v, float rscale) {
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
    uint32_t acc = 0;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const f16x2 h = __builtin_bit_cast(f16x2, w[i]);
        // fma(x, r, +0) = fl(x * r) (a product of -0 becomes +0, which rounds to the same integer): one
        // v_fma_mix_f32 reading the fp16 value, instead of a conversion and a multiplication
        float t0 = __builtin_amdgcn_fmed3f(__builtin_fmaf(static_cast<float>(h[0]), rscale, 0.0f), -8.0f, 7.0f);
        float t1 = __builtin_amdgcn_fmed3f(__builtin_fmaf(static_cast<float>(h[1]), rscale, 0.0f), -8.0f, 7.0f);
        acc += __float_as_uint(t0 + kMagic) << (8 * i);
        acc += __float_as_uint(t1 + kMagic) << (8 * i + 4);
    }
    return (acc - kMagicSum) ^ 0x88888888u;
}

__device__ __forceinline__ uint32_t absmax_bits(u32x4 v, uint32_t m) {
    m = pk_max_u16(m, v.x & 0x7FFF7FFFu);
    m = pk_max_u16(m, v.y & 0x7FFF7FFFu);
    m = pk_max_u16(m, v.z & 0x7FFF7FFFu);
    m = pk_max_u16(m, v.w & 0x7FFF7FFFu);
    return m;
}

__device__ __forceinline__ float absmax_exact(u32x4 v, float mx) {
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        mx = max_ignoring_nan(mx, fabsf(half_bits_to_float(w[i] & 0xFFFFu)));
        mx = max_ignoring_nan(mx, fabsf(half_bits_to_float(w[i] >> 16)));
    }
    return mx;
}

// scale = max > 0 ? (max / 7) * clip : 1, rounded to fp16 (token_scale_kernel).
__device__ __forceinline__ __half scale_from_absmax(float amax, float clip) {
    float s = amax > 0.0f ? (amax / 7.0f) * clip : 1.0f;
    return __float2half_rn(s);
}

__device__ __forceinline__ bool scale_is_ordinary(__half s) {
    uint32_t b = __half_as_ushort(s) & 0x7FFFu;
    return b != 0u && b < 0x7C00u;
}

// GELU, tanh approximation, on an fp16 value: the fp32 evaluation a framework
// applies to an fp16 tensor (the reference's FeedForward uses
// activation_fn="gelu-approximate", dit_block.py:56), rounded once to fp16:
//   u = sqrt(2/pi) * (x + 0.044715 * x^3),  gelu = 0.5 * x * (1 + tanh(u)).
// 0.5 * (1 + tanh(u)) is evaluated as 1 / (1 + exp(-2u)): no cancellation in the
// negative tail, so the fp32 result is a few ulp(fp32) from the exact value and
// the fp16 result is the correctly rounded one except next to a rounding boundary.
// +inf -> +inf, -inf -> NaN (= -inf * 0, as the formula gives), NaN -> NaN.
__device__ __forceinline__ float gelu_tanh_f32(float x) {
    // -2 * log2(e) * u = x * (c1 + c2 * x^2): the exponent of 2 in exp(-2u)
    constexpr float kC1 = -2.8853900817779268f * 0.7978845608028654f;
    constexpr float kC2 = kC1 * 0.044715f;
    const float a = x * __builtin_fmaf(kC2, x * x, kC1);
    const float e = __builtin_amdgcn_exp2f(a);
    return x * __builtin_amdgcn_rcpf(1.0f + e);
}

__device__ __forceinline__ uint32_t gelu_tanh_pair(uint32_t w) {
    const f16x2 h = __builtin_bit_cast(f16x2, w);
    f16x2 r;
    r[0] = static_cast<_Float16>(gelu_tanh_f32(static_cast<float>(h[0])));
    r[1] = static_cast<_Float16>(gelu_tanh_f32(static_cast<float>(h[1])));
    return __builtin_bit_cast(uint32_t, r);
}

template <int ACT>
__device__ __forceinline__ u32x4 apply_act(u32x4 v) {
    if (ACT == VDMQ_ACT_GELU_TANH) {
        v.x = gelu_tanh_pair(v.x);
        v.y = gelu_tanh_pair(v.y);
        v.z = gelu_tanh_pair(v.z);
        v.w = gelu_tanh_pair(v.w);
    }
    return v;
}

constexpr int kRowsPerBlock = 4; /* one wave per row */

template <bool STREAM>
__device__ __forceinline__ void store_word(uint32_t *p, uint32_t w) {
    if (STREAM)
        __builtin_nontemporal_store(w, p);
    else
        *p = w;
}

// Quantize a row held in registers (v[c] = elements 512c + 8*lane ... +7, zero
// beyond K): absmax, fp16 scale, nibbles, stores.
template <int NCH, bool STREAM_OUT>
__device__ __forceinline__ void quantize_held_row(const u32x4 (&v)[NCH], int lane, int64_t row, int Kp, float clip,
                                                  uint8_t *__restrict__ qact, __half *__restrict__ scale_h) {
    uint32_t m2 = 0;
#pragma unroll
    for (int c = 0; c < NCH; ++c) m2 = absmax_bits(v[c], m2);
    uint32_t m16 = (m2 & 0xFFFFu) > (m2 >> 16) ? (m2 & 0xFFFFu) : (m2 >> 16);
    m16 = wave_max(m16);

    uint32_t *dst = reinterpret_cast<uint32_t *>(qact + row * (Kp / 2));
    __half sh;
    bool fast = m16 < 0x7C00u; /* every element finite */
    if (fast) {
        sh = scale_from_absmax(half_bits_to_float(m16), clip);
        fast = scale_is_ordinary(sh);
    }
    if (fast) {
        const float rscale = 1.0f / __half2float(sh);
#pragma unroll
        for (int c = 0; c < NCH; ++c) {
            const int k0 = c * 512 + lane * 8;
            if (k0 < Kp) store_word<STREAM_OUT>(dst + c * 64 + lane, quantize_word_fast(v[c], rscale));
        }
    } else {
        float mx = 0.0f;
#pragma unroll
        for (int c = 0; c < NCH; ++c) mx = absmax_exact(v[c], mx);
        // fmaxf-style wave reduction (no NaN can be held in mx)
        mx = wave_max(mx);
        sh = scale_from_absmax(mx, clip);
        const float rscale = 1.0f / __half2float(sh);
#pragma unroll
        for (int c = 0; c < NCH; ++c) {
            const int k0 = c * 512 + lane * 8;
            if (k0 < Kp) store_word<STREAM_OUT>(dst + c * 64 + lane, quantize_word_exact(v[c], rscale));
        }
    }
    if (lane == 0) scale_h[row] = sh;
}

// The same, written as bf6 blocks (the operand form of the bf6 GEMM, see vdmq_bf6.hip): per row and 32
// consecutive k = 64 * kb + 32 * h + e one 192-bit string of six-bit E3M2 codes, stored by panels of 8 rows
// (bf6_piece in vdmq_internal.h).  A lane needs 32 consecutive k for that, but holds
// 8 per chunk: four chunks at a time go through a wave-private LDS buffer in k order (16 bytes of
// padding per 256 keep both the 16-byte writes and the 64-byte-per-lane reads free of bank
// conflicts) and come back as 32 consecutive fp16 per lane.  Those are scaled, rounded to integers
// (v_rndne_f32: half to even) and clamped exactly as in quantize_word_fast / quantize_word_exact,
// and the conversion instruction (v_cvt_scalef32_2xpk16_bf6_f32, or v_cvt_scalef32_pk32_bf6_f16 on the literal
// path) packs the 32 integers into the string with a scale of 16: the block holds q / 16, an E3M2 value for every
// q of [-8, 8] (code sign << 5 | |q|), so the conversion is exact.  Rows of the last row-block beyond M stay
// unwritten (the GEMM never stores them); K is padded to 128 with zeros.
typedef _Float16 f16x32 __attribute__((ext_vector_type(32)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef unsigned int u32x6 __attribute__((ext_vector_type(6)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));
constexpr int kBf6Rows = 8;                      /* rows (= waves) per workgroup of the bf6 quantizers */
constexpr int kTransposeBytes = 4 * (1024 + 64); /* four chunks plus padding, per wave */
constexpr int kStringsPerGroup = 64;             /* 2048 k = 64 strings of 32 k per row and group */

struct Bf6Scratch { /* LDS of one workgroup */
    uint8_t transpose[kBf6Rows][kTransposeBytes];
    // the strings of one group, 16-byte and 8-byte parts, [row][string] with one string of padding per row;
    // two copies, used alternately, so that one barrier per group is enough
    uint8_t part_a[2][kBf6Rows][(kStringsPerGroup + 1) * 16];
    uint8_t part_b[2][kBf6Rows][(kStringsPerGroup + 1) * 8];
};

// `valid`: the wave's row exists (a workgroup's waves all run this function -- it synchronises them --
// the ones past M on a copy of the last row, storing nothing).  `refill(c)` runs once chunk c of the
// row has gone to the transpose buffer and its registers are free: a workgroup that walks several
// row groups loads the next row's chunk there, so those loads overlap the rest of this row's
// conversion.  `phase` counts the groups this workgroup has staged (it picks the staging copy).
// Which row lengths take the walking form (a resident grid whose workgroups take row groups in turn, the next group's
// loads in flight under this group's conversion): rows longer than 8192, which leave room for one workgroup per CU
// only, and rows of at most 2048, whose groups are too little work for a workgroup of their own (K = 512...1536:
// +8...17 % at 32760 and 75600 rows; K = 3072: +2.5 % / -4 %; K = 4096: -6 %).
constexpr bool bf6_walks(int nch) { return nch >= 17 || nch <= 4; }
struct NoRefill {
    __device__ __forceinline__ void operator()(int) const {}
};
template <int NCH, class Refill>
__device__ __forceinline__ void quantize_held_row_bf6(u32x4 (&v)[NCH], int lane, int wave, int64_t row0, bool valid, int M, int Kb,
                                                      float clip, uint8_t *__restrict__ blocks, __half *__restrict__ scale_h,
                                                      bool stream_out, Bf6Scratch &lds, int &phase, Refill &&refill) {
    uint32_t m2 = 0;
#pragma unroll
    for (int c = 0; c < NCH; ++c) m2 = absmax_bits(v[c], m2);
    uint32_t m16 = (m2 & 0xFFFFu) > (m2 >> 16) ? (m2 & 0xFFFFu) : (m2 >> 16);
    m16 = wave_max(m16);
    __half sh;
    bool fast = m16 < 0x7C00u; /* every element finite */
    if (fast) {
        sh = scale_from_absmax(half_bits_to_float(m16), clip);
        fast = scale_is_ordinary(sh);
    }
    if (!fast) {
        float mx = 0.0f;
#pragma unroll
        for (int c = 0; c < NCH; ++c) mx = absmax_exact(v[c], mx);
        mx = wave_max(mx);
        sh = scale_from_absmax(mx, clip);
    }
    const float rscale = 1.0f / __half2float(sh);
    const bool fast_u = __builtin_amdgcn_readfirstlane(fast ? 1 : 0) != 0; /* the same in every lane: a scalar branch */
    if (lane == 0 && valid) scale_h[row0 + wave] = sh;

    const int kblocks = Kb / 64;
    uint8_t *tbuf = lds.transpose[wave];
    // the thread's share of the cooperative store: string t / 8 of row t % 8 -- eight consecutive
    // threads write the eight rows' parts of one string slot, 128 (and 64) contiguous bytes
    const int t = wave * kWaveSize + lane, srow = t % kBf6Rows, sidx = t / kBf6Rows;
    const int64_t grow = row0 + srow;
    constexpr int NG = (NCH + 3) / 4;
#pragma unroll
    for (int g = 0; g < NG; ++g) {
#pragma unroll
        for (int cc = 0; cc < 4; ++cc) {
            const int c = 4 * g + cc;
            const uint32_t off = cc * 1024 + lane * 16;
            *reinterpret_cast<u32x4 *>(tbuf + off + (off >> 8) * 16) = c < NCH ? v[c] : u32x4{0u, 0u, 0u, 0u};
        }
#pragma unroll
        for (int cc = 0; cc < 4; ++cc)
            if (4 * g + cc < NCH) refill(4 * g + cc);
        // (the LDS queue of a wave is in order: the reads below see the writes above)
        u32x4 tr[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) tr[u] = *reinterpret_cast<const u32x4 *>(tbuf + lane * 64 + u * 16 + (lane >> 2) * 16);
        // this lane's 32 consecutive k, 2048 g + 32 lane ..., become one 192-bit string
        u32x6 str;
        if (fast_u) {
            // the conversion from fp32 takes the even elements from one operand and the odd ones from the other:
            // the low and high halves of the words as they lie
            f32x16 even, odd;
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const uint32_t w[4] = {tr[u].x, tr[u].y, tr[u].z, tr[u].w};
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const f16x2 h = __builtin_bit_cast(f16x2, w[i]);
                    even[u * 4 + i] = __builtin_rintf(__builtin_amdgcn_fmed3f(__builtin_fmaf(static_cast<float>(h[0]), rscale, 0.0f), -8.0f, 7.0f));
                    odd[u * 4 + i] = __builtin_rintf(__builtin_amdgcn_fmed3f(__builtin_fmaf(static_cast<float>(h[1]), rscale, 0.0f), -8.0f, 7.0f));
                }
            }
            str = __builtin_amdgcn_cvt_scalef32_2xpk16_bf6_f32(even, odd, 16.0f);
        } else {
            f16x32 q;
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const uint32_t w[4] = {tr[u].x, tr[u].y, tr[u].z, tr[u].w};
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const f16x2 h = __builtin_bit_cast(f16x2, w[i]);
#pragma unroll
                    for (int e = 0; e < 2; ++e) { /* NaN -> 0, saturate, round half to even: cvt.rni + cvt.pack.sat of the reference */
                        const float p = static_cast<float>(h[e]) * rscale;
                        q[u * 8 + i * 2 + e] = static_cast<_Float16>(p != p ? 0.0f : (p >= 7.0f ? 7.0f : (p <= -8.0f ? -8.0f : __builtin_rintf(p))));
                    }
                }
            }
            str = __builtin_amdgcn_cvt_scalef32_pk32_bf6_f16(q, 16.0f);
        }
        // per-lane stores would scatter 16-byte pieces over 64 cache lines per instruction (measured: 2x
        // slower than the HBM-bound int4 quantizer): collect the workgroup's strings in LDS instead -- its
        // eight rows are one panel, whose 128-byte and 64-byte runs of one k-block are adjacent in memory
        const int copy = phase & 1;
        ++phase;
        *reinterpret_cast<u32x4 *>(lds.part_a[copy][wave] + lane * 16) = u32x4{str[0], str[1], str[2], str[3]};
        *reinterpret_cast<u32x2 *>(lds.part_b[copy][wave] + lane * 8) = u32x2{str[4], str[5]};
        __syncthreads(); /* also orders this group's writes after every thread's reads of the group before last */
        const int k0 = 2048 * g + 32 * sidx;
        if (k0 < Kb && grow < M) {
            const int kb = k0 >> 6, h = (k0 >> 5) & 1;
            const u32x4 part_a = *reinterpret_cast<const u32x4 *>(lds.part_a[copy][srow] + sidx * 16);
            const u32x2 part_b = *reinterpret_cast<const u32x2 *>(lds.part_b[copy][srow] + sidx * 8);
            u32x4 *dst_a = reinterpret_cast<u32x4 *>(blocks + bf6_piece(grow, kb, h, false, kblocks));
            u32x2 *dst_b = reinterpret_cast<u32x2 *>(blocks + bf6_piece(grow, kb, h, true, kblocks));
            if (stream_out) { /* the same for every thread of the launch */
                // (the empty statements keep the compiler from merging the two branches into plain stores)
                asm volatile("" ::: "memory");
                __builtin_nontemporal_store(part_a, dst_a);
                __builtin_nontemporal_store(part_b, dst_b);
                asm volatile("" ::: "memory");
            } else {
                *dst_a = part_a;
                *dst_b = part_b;
            }
        }
    }
}

// NCH = number of 512-element chunks (one 128-bit load per lane each) that
// cover the padded row.  STREAM_OUT: write the nibbles with non-temporal
// stores -- measured faster once the output no longer fits the 256 MB
// Infinity Cache (5.35 -> 5.9 TB/s at K = 13824, M = 75600), slower below.
// ACT: an elementwise activation applied to the row (in fp32, rounded to fp16)
// before it is quantized: the activation kernel between two linears, its write
// and the quantizer's re-read of its output are saved.
// FMT: 0 = native row-major int4 (Kp = K padded to the int8 GEMM's K step), 1 = bf6 blocks (Kp = K padded to 128)
template <int NCH, bool STREAM_OUT, int ACT, int FMT>
__global__ __launch_bounds__((FMT == 1 ? kBf6Rows : kRowsPerBlock) * kWaveSize) void quantize_rows_kernel(
    const __half *__restrict__ x, int64_t ldx, int M, int K, int Kp, float clip, uint8_t *__restrict__ qact,
    __half *__restrict__ scale_h, int stream_bf6) {
    constexpr int ROWS = FMT == 1 ? kBf6Rows : kRowsPerBlock;
    const int lane = threadIdx.x & (kWaveSize - 1), wave = threadIdx.x >> 6;
    if constexpr (FMT == 1) {
        // The workgroup walks row groups blockIdx.x, blockIdx.x + gridDim.x, ...: with the launcher's grid
        // (what the chip holds at once) the loads of the next group's rows are in flight while this
        // group's rows are converted -- a long row leaves room for one workgroup per CU only, whose load and
        // convert phases would otherwise alternate.
        __shared__ __attribute__((aligned(16))) Bf6Scratch scratch;
        const int groups = (M + ROWS - 1) / ROWS;
        auto row_ptr = [&](int group) {
            const int64_t r = static_cast<int64_t>(group) * ROWS + wave;
            return reinterpret_cast<const u32x4 *>(x + (r < M ? r : M - 1) * ldx); /* waves past M stay, on a copy of the last row */
        };
        auto load = [&](const u32x4 *src, int c) {
            return c * 512 + lane * 8 < K ? __builtin_nontemporal_load(src + c * 64 + lane) : u32x4{0u, 0u, 0u, 0u};
        };
        int group = blockIdx.x, phase = 0;
        u32x4 v[NCH];
        const u32x4 *src = row_ptr(group);
#pragma unroll
        for (int c = 0; c < NCH; ++c) v[c] = load(src, c);
        auto convert = [&](bool more) __attribute__((always_inline)) {
            if (ACT != VDMQ_ACT_NONE) {
#pragma unroll
                for (int c = 0; c < NCH; ++c)
                    if (c * 512 + lane * 8 < K) v[c] = apply_act<ACT>(v[c]);
            }
            const int64_t row0 = static_cast<int64_t>(group) * ROWS;
            const u32x4 *next = row_ptr(more ? group + gridDim.x : group);
            quantize_held_row_bf6<NCH>(v, lane, wave, row0, row0 + wave < M, M, Kp, clip, qact, scale_h, stream_bf6 != 0, scratch, phase,
                                       [&](int c) {
                                           if constexpr (bf6_walks(NCH))
                                               if (more) v[c] = load(next, c);
                                       });
        };
        if constexpr (bf6_walks(NCH)) {
            for (; group < groups; group += gridDim.x) convert(group + static_cast<int>(gridDim.x) < groups);
        } else {
            // short rows: one row group per workgroup -- several workgroups share a CU and overlap anyway
            convert(false);
        }
    } else {
        const int64_t row = static_cast<int64_t>(blockIdx.x) * ROWS + wave;
        if (row >= M) return;
        const u32x4 *src = reinterpret_cast<const u32x4 *>(x + row * ldx);
        u32x4 v[NCH];
#pragma unroll
        for (int c = 0; c < NCH; ++c) {
            const int k0 = c * 512 + lane * 8;
            v[c] = k0 < K ? apply_act<ACT>(__builtin_nontemporal_load(src + c * 64 + lane)) : u32x4{0u, 0u, 0u, 0u};
        }
        quantize_held_row<NCH, STREAM_OUT>(v, lane, row, Kp, clip, qact, scale_h);
    }
}

// Chunk counts the fused LayerNorm kernel is instantiated for (launch_ln_impl picks the first that covers the row):
// with NCH chunks the row is longer than the next smaller count, so the chunks below that one are complete in every
// lane and need no bounds test.
constexpr int ln_full_chunks(int nch) {
    constexpr int counts[] = {1, 2, 3, 4, 6, 10, 16, 32};
    int prev = 0;
    for (int n : counts)
        if (n < nch) prev = n;
    return prev;
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}

// LayerNorm over the row (fp32 statistics, no affine) followed by the block's
// modulation, fused in front of the quantizer -- the producer of the attn1 and
// FFN-up inputs (dit_block.py:100, :110 of the reference):
//   VDMQ_LN_MODULATE  h = (fp16(LN(x)) * (1 + a)) + b   with a = scale, b = shift, every
//                     operation a correctly rounded fp16 operation, as the reference's
//                     fp16 tensor arithmetic after FP32LayerNorm's cast back to fp16
//   VDMQ_LN_AFFINE    h = fp16(LN(x) * a + b)           with a = weight, b = bias, in
//                     fp32 with one rounding (FP32LayerNorm with elementwise_affine, norm2)
// Row m takes vector row m / rows_per_vec of a and b (stride ldv elements): one
// vector per batch element, or one per token.  EMIT_H writes h itself instead of
// quantizing it (the same arithmetic: the checker's view of h).
template <int NCH, int LNMODE, bool EMIT_H, int FMT>
__global__ __launch_bounds__((FMT == 1 ? kBf6Rows : kRowsPerBlock) * kWaveSize) void ln_quantize_rows_kernel(
    const __half *__restrict__ x, int64_t ldx, int M, int K, int Kp, float eps, const __half *__restrict__ va,
    const __half *__restrict__ vb, int64_t ldv, int rows_per_vec, float clip, uint8_t *__restrict__ qact,
    __half *__restrict__ scale_h, __half *__restrict__ h_out, int64_t ldh, int stream_bf6) {
    constexpr int ROWS = FMT == 1 ? kBf6Rows : kRowsPerBlock;
    const int lane = threadIdx.x & (kWaveSize - 1), wave = threadIdx.x >> 6;
    const int64_t row0 = static_cast<int64_t>(blockIdx.x) * ROWS;
    int64_t row = row0 + wave;
    const bool valid = row < M;
    if (!valid) {
        if (FMT == 0) return;
        row = M - 1; /* the bf6 tail synchronises the workgroup: stay, on a copy of the last row */
    }
    const u32x4 *src = reinterpret_cast<const u32x4 *>(x + row * ldx);
    const int64_t vrow = (row / rows_per_vec) * ldv;
    const u32x4 *pa = reinterpret_cast<const u32x4 *>(va + vrow), *pb = reinterpret_cast<const u32x4 *>(vb + vrow);

    u32x4 v[NCH];
    float sum = 0.0f;
    float one = 1.0f; /* a multiplier the compiler cannot see through: fma(x, one, y) stays a fused multiply-add */
    asm volatile("" : "+s"(one));
#pragma unroll
    for (int c = 0; c < NCH; ++c) {
        const int k0 = c * 512 + lane * 8;
        v[c] = c < ln_full_chunks(NCH) || k0 < K ? __builtin_nontemporal_load(src + c * 64 + lane) : u32x4{0u, 0u, 0u, 0u};
        const uint32_t w[4] = {v[c].x, v[c].y, v[c].z, v[c].w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const f16x2 h = __builtin_bit_cast(f16x2, w[i]);
            // fma(x, 1, s) = fl(x + s) as one v_fma_mix_f32, which reads the fp16 value directly (padding adds zeros)
            sum = __builtin_fmaf(static_cast<float>(h[0]), one, sum);
            sum = __builtin_fmaf(static_cast<float>(h[1]), one, sum);
        }
    }
    const float mean = wave_sum(sum) / static_cast<float>(K);
    // Each pass converts the fp16 row again: the compiler would otherwise keep the 8 * NCH converted floats of one
    // pass for the next (80 registers for a 5120-wide row, a workgroup per CU less); the empty asm makes the row
    // a new value for it.
#pragma unroll
    for (int c = 0; c < NCH; ++c) asm volatile("" : "+v"(v[c]));
    float sq = 0.0f;
#pragma unroll
    for (int c = 0; c < NCH; ++c) {
        const int k0 = c * 512 + lane * 8;
        if (c < ln_full_chunks(NCH) || k0 < K) {
            const uint32_t w[4] = {v[c].x, v[c].y, v[c].z, v[c].w};
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const f16x2 h = __builtin_bit_cast(f16x2, w[i]);
                const float d0 = __builtin_fmaf(static_cast<float>(h[0]), one, -mean), d1 = __builtin_fmaf(static_cast<float>(h[1]), one, -mean);
                sq = __builtin_fmaf(d0, d0, sq);
                sq = __builtin_fmaf(d1, d1, sq);
            }
        }
    }
    const float rstd = 1.0f / __builtin_sqrtf(wave_sum(sq) / static_cast<float>(K) + eps);
#pragma unroll
    for (int c = 0; c < NCH; ++c) asm volatile("" : "+v"(v[c]));

#pragma unroll
    for (int c = 0; c < NCH; ++c) {
        const int k0 = c * 512 + lane * 8;
        if (c < ln_full_chunks(NCH) || k0 < K) {
            const u32x4 a4 = pa[c * 64 + lane], b4 = pb[c * 64 + lane];
            const uint32_t w[4] = {v[c].x, v[c].y, v[c].z, v[c].w};
            const uint32_t aw[4] = {a4.x, a4.y, a4.z, a4.w}, bw[4] = {b4.x, b4.y, b4.z, b4.w};
            uint32_t o[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const f16x2 h = __builtin_bit_cast(f16x2, w[i]);
                const f16x2 a = __builtin_bit_cast(f16x2, aw[i]), b = __builtin_bit_cast(f16x2, bw[i]);
                const float n0 = __builtin_fmaf(static_cast<float>(h[0]), one, -mean) * rstd;
                const float n1 = __builtin_fmaf(static_cast<float>(h[1]), one, -mean) * rstd;
                f16x2 r;
                if (LNMODE == VDMQ_LN_MODULATE) {
                    const f16x2 ln = {static_cast<_Float16>(n0), static_cast<_Float16>(n1)};
                    const f16x2 one = {static_cast<_Float16>(1.0f), static_cast<_Float16>(1.0f)};
                    r = ln * (one + a) + b; /* three packed fp16 operations, each rounded (no contraction) */
                } else {
                    r[0] = static_cast<_Float16>(n0 * static_cast<float>(a[0]) + static_cast<float>(b[0]));
                    r[1] = static_cast<_Float16>(n1 * static_cast<float>(a[1]) + static_cast<float>(b[1]));
                }
                o[i] = __builtin_bit_cast(uint32_t, r);
            }
            v[c] = u32x4{o[0], o[1], o[2], o[3]};
        }
    }
    if (EMIT_H) {
        u32x4 *dst = reinterpret_cast<u32x4 *>(h_out + row * ldh);
#pragma unroll
        for (int c = 0; c < NCH; ++c) {
            const int k0 = c * 512 + lane * 8;
            if (k0 < K) dst[c * 64 + lane] = v[c];
        }
        return;
    }
    if (FMT == 1) {
        __shared__ __attribute__((aligned(16))) Bf6Scratch scratch;
        int phase = 0;
        quantize_held_row_bf6<NCH>(v, lane, wave, row0, valid, M, Kp, clip, qact, scale_h, stream_bf6 != 0, scratch, phase, NoRefill{});
    } else {
        quantize_held_row<NCH, false>(v, lane, row, Kp, clip, qact, scale_h);
    }
}

// Any K: two passes over the row (the second one is served by the caches).
template <int ACT>
__global__ __launch_bounds__(kRowsPerBlock * kWaveSize) void quantize_rows_anyk_kernel(const __half *__restrict__ x, int64_t ldx,
                                                                                       int M, int K, int Kp, float clip,
                                                                                       uint8_t *__restrict__ qact,
                                                                                       __half *__restrict__ scale_h) {
    const int lane = threadIdx.x & (kWaveSize - 1);
    const int64_t row = static_cast<int64_t>(blockIdx.x) * kRowsPerBlock + (threadIdx.x >> 6);
    if (row >= M) return;
    const u32x4 *src = reinterpret_cast<const u32x4 *>(x + row * ldx);
    float mx = 0.0f;
    for (int k0 = lane * 8; k0 < K; k0 += 512) mx = absmax_exact(apply_act<ACT>(src[k0 / 8]), mx);
    mx = wave_max(mx);
    const __half sh = scale_from_absmax(mx, clip);
    const float rscale = 1.0f / __half2float(sh);
    uint32_t *dst = reinterpret_cast<uint32_t *>(qact + row * (Kp / 2));
    for (int k0 = lane * 8; k0 < Kp; k0 += 512) {
        u32x4 v = k0 < K ? apply_act<ACT>(src[k0 / 8]) : u32x4{0u, 0u, 0u, 0u};
        dst[k0 / 8] = quantize_word_exact(v, rscale);
    }
    if (lane == 0) scale_h[row] = sh;
}

// Per-row scale only (weights: quantize_weight_per_channel's first launch).
__global__ __launch_bounds__(kRowsPerBlock * kWaveSize) void row_scale_kernel(const __half *__restrict__ x, int64_t rows, int K,
                                                                              float clip, __half *__restrict__ scale_h) {
    const int lane = threadIdx.x & (kWaveSize - 1);
    const int64_t row = static_cast<int64_t>(blockIdx.x) * kRowsPerBlock + (threadIdx.x >> 6);
    if (row >= rows) return;
    const u32x4 *src = reinterpret_cast<const u32x4 *>(x + row * static_cast<int64_t>(K));
    float mx = 0.0f;
    for (int k0 = lane * 8; k0 < K; k0 += 512) mx = absmax_exact(src[k0 / 8], mx);
    mx = wave_max(mx);
    if (lane == 0) scale_h[row] = scale_from_absmax(mx, clip);
}

// Quantize rows with caller-provided fp16 scales into the native layout
// (weights: quantize_warp_static_scale, vdm_w4a4_kernel.cu:296-338).
__global__ __launch_bounds__(256) void quantize_given_scale_kernel(const __half *__restrict__ x, const __half *__restrict__ scale_h,
                                                                   int64_t rows, int K, int Kp, uint8_t *__restrict__ q) {
    const int64_t words_per_row = Kp / 8;
    const int64_t idx = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (idx >= rows * words_per_row) return;
    const int64_t row = idx / words_per_row;
    const int k0 = static_cast<int>(idx % words_per_row) * 8;
    u32x4 v = k0 < K ? *reinterpret_cast<const u32x4 *>(x + row * K + k0) : u32x4{0u, 0u, 0u, 0u};
    const float rscale = 1.0f / __half2float(scale_h[row]);
    reinterpret_cast<uint32_t *>(q)[idx] = quantize_word_exact(v, rscale);
}

constexpr int64_t kStreamOutBytes = int64_t(224) << 20; /* outputs larger than this bypass the caches */
// The same for the bf6 blocks, judged by the quantizer and the GEMM that reads its output together: streamed stores
// cost the GEMM the part of its operand that plain stores leave in the Infinity Cache (38 MB and 63 MB of blocks:
// the pair 3 % and 2 % slower), and spare it the wait for the dirty lines of a large one (220 MB, 290 MB, 780 MB:
// the pair 3 %, 0.7 % and 0.7 % faster).
constexpr int64_t kStreamOutBytesBf6 = int64_t(128) << 20;
int stream_bf6(int64_t M, int64_t K) { return bf6_bytes(M, K) > kStreamOutBytesBf6 ? 1 : 0; }

// Workgroups of `kernel` the current device runs at once (CUs x workgroups per CU), or -1.  The answer is
// kept per device in `cache` (one array per kernel, zero-initialised): the occupancy query costs tens of
// microseconds, which a launch on an idle stream would show.
constexpr int kMaxDevices = 64;
int64_t resident_workgroups(const void *kernel, int threads, int (&cache)[kMaxDevices]) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return -1;
    if (cache[dev] > 0) return cache[dev];
    int cus = 0, per_cu = 0;
    if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess ||
        hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kernel, threads, 0) != hipSuccess || cus <= 0 || per_cu <= 0) {
        (void)hipGetLastError();
        return -1;
    }
    cache[dev] = cus * per_cu; /* racing first calls store the same value */
    return cache[dev];
}

template <int NCH, int ACT>
int launch_reg(const __half *x, int64_t M, int64_t K, int64_t ldx, float clip, int fmt, uint8_t *qact, __half *scale_h, hipStream_t s) {
    const dim3 grid(static_cast<unsigned>(ceil_div(M, kRowsPerBlock))), block(kRowsPerBlock * kWaveSize);
    if (fmt == 1) {
        const int64_t groups = ceil_div(M, kBf6Rows);
        static int cache[kMaxDevices];
        const int64_t resident = !bf6_walks(NCH) ? groups
                                 : resident_workgroups(reinterpret_cast<const void *>(&quantize_rows_kernel<NCH, false, ACT, 1>),
                                                       kBf6Rows * kWaveSize, cache);
        if (resident <= 0) return fail(VDMQ_ELAUNCH, "quantize_rows_kernel: the occupancy query for the current device failed");
        hipLaunchKernelGGL((quantize_rows_kernel<NCH, false, ACT, 1>), dim3(static_cast<unsigned>(!bf6_walks(NCH) || groups < resident ? groups : resident)),
                           dim3(kBf6Rows * kWaveSize), 0, s, x, ldx, static_cast<int>(M), static_cast<int>(K),
                           static_cast<int>(bf6_kblocks(K) * 64), clip, qact, scale_h, stream_bf6(M, K));
    }
    else if (M * (k_padded(K) / 2) > kStreamOutBytes)
        hipLaunchKernelGGL((quantize_rows_kernel<NCH, true, ACT, 0>), grid, block, 0, s, x, ldx, static_cast<int>(M), static_cast<int>(K),
                           static_cast<int>(k_padded(K)), clip, qact, scale_h, 0);
    else
        hipLaunchKernelGGL((quantize_rows_kernel<NCH, false, ACT, 0>), grid, block, 0, s, x, ldx, static_cast<int>(M), static_cast<int>(K),
                           static_cast<int>(k_padded(K)), clip, qact, scale_h, 0);
    return check_launch("quantize_rows_kernel");
}

template <int ACT>
int launch_quantize_act_impl(const __half *x, int64_t M, int64_t K, int64_t ldx, float clip, int fmt, uint8_t *qact, __half *scale_h,
                             hipStream_t s) {
    const int64_t nch = ceil_div(k_padded(K), 512);
#define VDMQ_CASE(n) \
    if (nch <= n) return launch_reg<n, ACT>(x, M, K, ldx, clip, fmt, qact, scale_h, s)
    // Rows are held in registers, so the chunk count is a template parameter; a row runs on the first count that
    // covers it (loads beyond K are predicated off: the spare chunks cost registers, not bytes).  Instantiated: what
    // the Wan models' linears need -- K = 1536, 3072, 5120 (3, 6, 10), the FFN widths 8960, 13824 and 14336 (18, 28,
    // 28) -- the small counts, and a sparse cover of the rest up to K = 16384.
    VDMQ_CASE(1);
    VDMQ_CASE(2);
    VDMQ_CASE(3);
    VDMQ_CASE(4);
    VDMQ_CASE(6);
    VDMQ_CASE(10);
    VDMQ_CASE(14);
    VDMQ_CASE(18);
    VDMQ_CASE(24);
    VDMQ_CASE(28);
    VDMQ_CASE(32);
#undef VDMQ_CASE
    if (fmt == 1) return fail(VDMQ_ESHAPE, "the bf6 quantizer needs K <= 16384 (got %lld)", (long long)K);
    const unsigned grid = static_cast<unsigned>(ceil_div(M, kRowsPerBlock));
    hipLaunchKernelGGL(quantize_rows_anyk_kernel<ACT>, dim3(grid), dim3(kRowsPerBlock * kWaveSize), 0, s, x, ldx, static_cast<int>(M),
                       static_cast<int>(K), static_cast<int>(k_padded(K)), clip, qact, scale_h);
    return check_launch("quantize_rows_anyk_kernel");
}

template <int NCH, int LNMODE>
int launch_ln_reg(const __half *x, int64_t M, int64_t K, int64_t ldx, float eps, const __half *va, const __half *vb, int64_t ldv,
                  int64_t rows_per_vec, float clip, int fmt, uint8_t *qact, __half *scale_h, __half *h_out, int64_t ldh, hipStream_t s) {
    const dim3 grid(static_cast<unsigned>(ceil_div(M, kRowsPerBlock))), block(kRowsPerBlock * kWaveSize);
    if (h_out != nullptr)
        hipLaunchKernelGGL((ln_quantize_rows_kernel<NCH, LNMODE, true, 0>), grid, block, 0, s, x, ldx, static_cast<int>(M), static_cast<int>(K),
                           static_cast<int>(k_padded(K)), eps, va, vb, ldv, static_cast<int>(rows_per_vec), clip, qact, scale_h, h_out, ldh, 0);
    else if (fmt == 1)
        hipLaunchKernelGGL((ln_quantize_rows_kernel<NCH, LNMODE, false, 1>), dim3(static_cast<unsigned>(ceil_div(M, kBf6Rows))),
                           dim3(kBf6Rows * kWaveSize), 0, s, x, ldx, static_cast<int>(M), static_cast<int>(K),
                           static_cast<int>(bf6_kblocks(K) * 64), eps, va, vb, ldv, static_cast<int>(rows_per_vec), clip, qact, scale_h, h_out, ldh,
                           stream_bf6(M, K));
    else
        hipLaunchKernelGGL((ln_quantize_rows_kernel<NCH, LNMODE, false, 0>), grid, block, 0, s, x, ldx, static_cast<int>(M), static_cast<int>(K),
                           static_cast<int>(k_padded(K)), eps, va, vb, ldv, static_cast<int>(rows_per_vec), clip, qact, scale_h, h_out, ldh, 0);
    return check_launch("ln_quantize_rows_kernel");
}

template <int LNMODE>
int launch_ln_impl(const __half *x, int64_t M, int64_t K, int64_t ldx, float eps, const __half *va, const __half *vb, int64_t ldv,
                   int64_t rows_per_vec, float clip, int fmt, uint8_t *qact, __half *scale_h, __half *h_out, int64_t ldh, hipStream_t s) {
    const int64_t nch = ceil_div(k_padded(K), 512);
#define VDMQ_CASE(n) \
    if (nch <= n) return launch_ln_reg<n, LNMODE>(x, M, K, ldx, eps, va, vb, ldv, rows_per_vec, clip, fmt, qact, scale_h, h_out, ldh, s)
    // (the counts of ln_full_chunks: the LayerNorm runs over a model's width -- 1536, 3072, 5120: 3, 6, 10)
    VDMQ_CASE(1);
    VDMQ_CASE(2);
    VDMQ_CASE(3);
    VDMQ_CASE(4);
    VDMQ_CASE(6);
    VDMQ_CASE(10);
    VDMQ_CASE(16);
    VDMQ_CASE(32);
#undef VDMQ_CASE
    return fail(VDMQ_ESHAPE, "the fused LayerNorm needs K <= 16384 (got %lld)", (long long)K);
}

__global__ __launch_bounds__(256) void gelu_tanh_kernel(const uint32_t *__restrict__ x, uint32_t *__restrict__ y, int64_t pairs) {
    const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i < pairs) y[i] = gelu_tanh_pair(x[i]);
}

}  // namespace

int launch_quantize_act(const __half *x, int64_t M, int64_t K, int64_t ldx, float clip, int act, int fmt, uint8_t *qact,
                        __half *scale_h, hipStream_t s) {
    if (M == 0) return VDMQ_OK;
    if (act == VDMQ_ACT_GELU_TANH) return launch_quantize_act_impl<VDMQ_ACT_GELU_TANH>(x, M, K, ldx, clip, fmt, qact, scale_h, s);
    return launch_quantize_act_impl<VDMQ_ACT_NONE>(x, M, K, ldx, clip, fmt, qact, scale_h, s);
}

int launch_ln_quantize(const __half *x, int64_t M, int64_t K, int64_t ldx, float eps, int ln_mode, const __half *va, const __half *vb,
                       int64_t ldv, int64_t rows_per_vec, float clip, int fmt, uint8_t *qact, __half *scale_h, __half *h_out, int64_t ldh,
                       hipStream_t s) {
    if (M == 0) return VDMQ_OK;
    if (ln_mode == VDMQ_LN_MODULATE)
        return launch_ln_impl<VDMQ_LN_MODULATE>(x, M, K, ldx, eps, va, vb, ldv, rows_per_vec, clip, fmt, qact, scale_h, h_out, ldh, s);
    return launch_ln_impl<VDMQ_LN_AFFINE>(x, M, K, ldx, eps, va, vb, ldv, rows_per_vec, clip, fmt, qact, scale_h, h_out, ldh, s);
}

int launch_gelu_tanh(const __half *x, __half *y, int64_t n, hipStream_t s) {
    const int64_t pairs = n / 2;
    if (pairs == 0) return VDMQ_OK;
    hipLaunchKernelGGL(gelu_tanh_kernel, dim3(static_cast<unsigned>(ceil_div(pairs, 256))), dim3(256), 0, s,
                       reinterpret_cast<const uint32_t *>(x), reinterpret_cast<uint32_t *>(y), pairs);
    return check_launch("gelu_tanh_kernel");
}

int launch_row_scale(const __half *x, int64_t rows, int64_t K, float clip, __half *scale_h, hipStream_t s) {
    if (rows == 0) return VDMQ_OK;
    hipLaunchKernelGGL(row_scale_kernel, dim3(static_cast<unsigned>(ceil_div(rows, kRowsPerBlock))),
                       dim3(kRowsPerBlock * kWaveSize), 0, s, x, rows, static_cast<int>(K), clip, scale_h);
    return check_launch("row_scale_kernel");
}

int launch_quantize_given_scale(const __half *x, const __half *scale_h, int64_t rows, int64_t K, uint8_t *q, hipStream_t s) {
    if (rows == 0) return VDMQ_OK;
    const int64_t total = rows * (k_padded(K) / 8);
    hipLaunchKernelGGL(quantize_given_scale_kernel, dim3(static_cast<unsigned>(ceil_div(total, 256))), dim3(256), 0, s, x, scale_h,
                       rows, static_cast<int>(K), static_cast<int>(k_padded(K)), q);
    return check_launch("quantize_given_scale_kernel");
}

}  // namespace vdmq
