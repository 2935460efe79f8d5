// Relayouts between the checkpoint's v1 buffers and the native row-major ones.
//
// Both layouts keep eight consecutive-k int4 values in one 32-bit word with
// element e in nibble e, so every relayout is a permutation of 32-bit words.
// The v1 word order is the one the reference's CUDA packers emit
// (vdm_w4a4_kernel.cu:483-551): 16-byte groups indexed
//   weights      ((bn*KG + bk)*8 + tile)*32 + lane            (:545)
//   activations  (((bm*KG + bk)*8 + warp)*2 + tile)*32 + lane (:511)
// whose four words are, with g = lane/4 and t = lane%4, the k-ranges
// [8t, 8t+8) and [32+8t, 32+8t+8) of rows g and g+8 of a 16-row tile; the
// weight packer orders them (row g: k-lo, k-hi; row g+8: k-lo, k-hi)
// (:542-544), the activation packer (k-lo: row g, row g+8; k-hi: row g, g+8).
// These kernels run once per module or per API-compatibility call; they are
// not on the timed path.
#include "vdmq_internal.h"

namespace vdmq {
namespace {

struct WordCoord {
    int64_t row;
    int k0;
};

__device__ __forceinline__ WordCoord weight_v1_word(int64_t widx, int KG) {
    const int comp = static_cast<int>(widx & 3);
    const int64_t u = widx >> 2;
    const int lane = static_cast<int>(u & 31);
    const int tile = static_cast<int>((u >> 5) & 7);
    const int64_t blk = u >> 8;
    const int bk = static_cast<int>(blk % KG);
    const int64_t bn = blk / KG;
    const int g = lane >> 2, t = lane & 3;
    const int hi_n = comp >> 1, khalf = comp & 1;
    return {bn * 128 + tile * 16 + hi_n * 8 + g, bk * 64 + khalf * 32 + t * 8};
}

__device__ __forceinline__ WordCoord act_v1_word(int64_t widx, int KG) {
    const int comp = static_cast<int>(widx & 3);
    const int64_t u = widx >> 2;
    const int lane = static_cast<int>(u & 31);
    const int tile = static_cast<int>((u >> 5) & 1);
    const int warp = static_cast<int>((u >> 6) & 7);
    const int64_t blk = u >> 9;
    const int bk = static_cast<int>(blk % KG);
    const int64_t bm = blk / KG;
    const int g = lane >> 2, t = lane & 3;
    const int khalf = comp >> 1, hi_m = comp & 1;
    return {bm * 256 + warp * 32 + tile * 16 + hi_m * 8 + g, bk * 64 + khalf * 32 + t * 8};
}

template <bool TO_NATIVE>
__global__ __launch_bounds__(256) void weight_relayout_kernel(const uint32_t *__restrict__ src, uint32_t *__restrict__ dst, int64_t N,
                                                              int K, int Kp) {
    const int64_t widx = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (TO_NATIVE) {
        // one thread per native word so that the zero padding is written too
        const int64_t wpr = Kp / 8;
        if (widx >= N * wpr) return;
        const int64_t n = widx / wpr;
        const int k0 = static_cast<int>(widx % wpr) * 8;
        uint32_t v = 0;
        if (k0 < K) {
            const int KG = K / 64;
            const int bk = k0 >> 6, kk = k0 & 63, khalf = kk >> 5, t = (kk >> 3) & 3;
            const int r = static_cast<int>(n & 15), g = r & 7, hi_n = r >> 3;
            const int64_t u = ((n >> 7) * KG + bk) * 256 + ((n >> 4) & 7) * 32 + (4 * g + t);
            v = src[u * 4 + 2 * hi_n + khalf];
        }
        dst[widx] = v;
    } else {
        if (widx >= N * (K / 8)) return;
        const WordCoord c = weight_v1_word(widx, K / 64);
        dst[widx] = src[c.row * (Kp / 8) + c.k0 / 8];
    }
}

// packed v1 scale index of (channel n, k-group bk): pack_wscales, :286-294, :550
__device__ __forceinline__ int64_t wscale_v1_index(int64_t n, int bk, int KG) {
    const int j = static_cast<int>((n >> 4) & 7), r = static_cast<int>(n & 15);
    return (((n >> 7) * KG + bk) * 32 + 4 * j + ((r & 7) >> 1)) * 4 + 2 * (r >> 3) + (r & 1);
}

// v1 scale index of (token row m, k-group bk): pack_ascales, :276-284, :514-515
__device__ __forceinline__ int64_t ascale_v1_index(int64_t m, int bk, int KG) {
    const int warp = static_cast<int>((m >> 5) & 7), i = static_cast<int>((m >> 4) & 1), r = static_cast<int>(m & 15);
    return ((((m >> 8) * KG + bk) * 8 + warp) * 16 + 8 * i + (r & 7)) * 2 + (r >> 3);
}

__global__ __launch_bounds__(256) void wscale_to_plain_kernel(const __half *__restrict__ packed, __half *__restrict__ plain, int64_t N,
                                                              int KG) {
    const int64_t n = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (n < N) plain[n] = packed[wscale_v1_index(n, 0, KG)];
}

__global__ __launch_bounds__(256) void wscale_to_v1_kernel(const __half *__restrict__ plain, __half *__restrict__ packed, int64_t N,
                                                           int KG) {
    const int64_t idx = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (idx >= N * KG) return;
    const int64_t n = idx / KG;
    packed[wscale_v1_index(n, static_cast<int>(idx % KG), KG)] = plain[n];
}

__global__ __launch_bounds__(256) void act_to_v1_kernel(const uint32_t *__restrict__ qact, const __half *__restrict__ scale_h, int64_t M,
                                                        int64_t PM, int K, int Kp, uint32_t *__restrict__ qact_v1,
                                                        __half *__restrict__ ascales_v1) {
    const int64_t widx = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    const int KG = K / 64;
    if (widx < PM * (K / 8)) {
        const WordCoord c = act_v1_word(widx, KG);
        qact_v1[widx] = c.row < M ? qact[c.row * (Kp / 8) + c.k0 / 8] : 0u;
    }
    if (widx < PM * KG) {
        const int64_t m = widx / KG;
        ascales_v1[ascale_v1_index(m, static_cast<int>(widx % KG), KG)] = m < M ? scale_h[m] : __float2half_rn(1.0f);
    }
}

__global__ __launch_bounds__(256) void act_to_native_kernel(const uint32_t *__restrict__ qact_v1, const __half *__restrict__ ascales_v1,
                                                            int64_t M, int K, int Kp, uint32_t *__restrict__ qact,
                                                            __half *__restrict__ scale_h) {
    const int64_t widx = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    const int KG = K / 64;
    const int64_t wpr = Kp / 8;
    if (widx < M * wpr) {
        const int64_t m = widx / wpr;
        const int k0 = static_cast<int>(widx % wpr) * 8;
        uint32_t v = 0;
        if (k0 < K) {
            const int bk = k0 >> 6, kk = k0 & 63, khalf = kk >> 5, t = (kk >> 3) & 3;
            const int r = static_cast<int>(m & 15), g = r & 7, hi_m = r >> 3;
            const int64_t u = ((((m >> 8) * KG + bk) * 8 + ((m >> 5) & 7)) * 2 + ((m >> 4) & 1)) * 32 + (4 * g + t);
            v = qact_v1[u * 4 + 2 * khalf + hi_m];
        }
        qact[widx] = v;
    }
    if (widx < M) scale_h[widx] = ascales_v1[ascale_v1_index(widx, 0, KG)];
}

// Plain copy with 128-bit accesses (non-temporal loads, like the quantizer's):
// a kernel of known traffic to scale hardware counters by.
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
__global__ __launch_bounds__(256) void copy_u128_kernel(const u32x4 *__restrict__ src, u32x4 *__restrict__ dst, int64_t n) {
    const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i < n) dst[i] = __builtin_nontemporal_load(src + i);
}

// Streaming probe with another mix of reads and writes than the copy's 1 : 1: a wave loads READS consecutive
// kilobytes of src (one per instruction, 16 bytes per lane) and stores WRITES consecutive kilobytes of dst derived
// from all of them -- the quantizers' pattern: a wave reads a contiguous row and writes a shorter contiguous one.
// With 8 : 3 it moves the A4 quantizer's 2 bytes read per 3/4 byte written (6-bit operand blocks), with 4 : 1 the
// int4 rows' ratio, and does nothing else: what it sustains is what the memory system gives a kernel of that mix.
template <int READS, int WRITES>
__global__ __launch_bounds__(256) void stream_mix_kernel(const u32x4 *__restrict__ src, u32x4 *__restrict__ dst, int64_t threads) {
    const int64_t t = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (t >= threads) return;
    const int64_t wave = t >> 6, lane = t & 63;
    src += wave * READS * 64 + lane;
    dst += wave * WRITES * 64 + lane;
    u32x4 v[READS];
#pragma unroll
    for (int j = 0; j < READS; ++j) v[j] = __builtin_nontemporal_load(src + j * 64);
    u32x4 x = v[0];
#pragma unroll
    for (int j = 1; j < READS; ++j) x ^= v[j];
    if (WRITES == 0) asm volatile("" ::"v"(x.x), "v"(x.y), "v"(x.z), "v"(x.w)); /* (keeps the loads of a read-only run) */
#pragma unroll
    for (int j = 0; j < WRITES; ++j) {
        __builtin_nontemporal_store(x, dst + j * 64);
        x += u32x4{1u, 1u, 1u, 1u};
    }
}

unsigned blocks_for(int64_t n) { return static_cast<unsigned>(ceil_div(n > 0 ? n : 1, 256)); }

}  // namespace

int launch_copy_u128(const void *src, void *dst, int64_t bytes, hipStream_t s) {
    const int64_t n = bytes / 16;
    if (n == 0) return VDMQ_OK;
    hipLaunchKernelGGL(copy_u128_kernel, dim3(blocks_for(n)), dim3(256), 0, s, static_cast<const u32x4 *>(src),
                       static_cast<u32x4 *>(dst), n);
    return check_launch("copy_u128_kernel");
}

int launch_stream_mix(const void *src, void *dst, int64_t threads, int reads, int writes, hipStream_t s) {
    if (threads == 0) return VDMQ_OK;
    const u32x4 *in = static_cast<const u32x4 *>(src);
    u32x4 *out = static_cast<u32x4 *>(dst);
    if (reads == 8 && writes == 3)
        hipLaunchKernelGGL((stream_mix_kernel<8, 3>), dim3(blocks_for(threads)), dim3(256), 0, s, in, out, threads);
    else if (reads == 4 && writes == 1)
        hipLaunchKernelGGL((stream_mix_kernel<4, 1>), dim3(blocks_for(threads)), dim3(256), 0, s, in, out, threads);
    else if (reads == 1 && writes == 1)
        hipLaunchKernelGGL((stream_mix_kernel<1, 1>), dim3(blocks_for(threads)), dim3(256), 0, s, in, out, threads);
    else if (reads == 4 && writes == 0)
        hipLaunchKernelGGL((stream_mix_kernel<4, 0>), dim3(blocks_for(threads)), dim3(256), 0, s, in, out, threads);
    else
        return fail(VDMQ_EINVAL, "stream probe mixes: 8 : 3, 4 : 1, 1 : 1, 4 : 0 (got %d : %d)", reads, writes);
    return check_launch("stream_mix_kernel");
}

int launch_weight_relayout(const void *src, void *dst, int64_t N, int64_t K, bool to_native, hipStream_t s) {
    const int Kp = static_cast<int>(k_padded(K));
    if (to_native) {
        hipLaunchKernelGGL(weight_relayout_kernel<true>, dim3(blocks_for(N * (Kp / 8))), dim3(256), 0, s,
                           static_cast<const uint32_t *>(src), static_cast<uint32_t *>(dst), N, static_cast<int>(K), Kp);
    } else {
        hipLaunchKernelGGL(weight_relayout_kernel<false>, dim3(blocks_for(N * (K / 8))), dim3(256), 0, s,
                           static_cast<const uint32_t *>(src), static_cast<uint32_t *>(dst), N, static_cast<int>(K), Kp);
    }
    return check_launch("weight_relayout_kernel");
}

int launch_wscale_relayout(const void *src, void *dst, int64_t N, int64_t K, bool to_plain, hipStream_t s) {
    const int KG = static_cast<int>(K / 64);
    if (to_plain) {
        hipLaunchKernelGGL(wscale_to_plain_kernel, dim3(blocks_for(N)), dim3(256), 0, s, static_cast<const __half *>(src),
                           static_cast<__half *>(dst), N, KG);
    } else {
        hipLaunchKernelGGL(wscale_to_v1_kernel, dim3(blocks_for(N * KG)), dim3(256), 0, s, static_cast<const __half *>(src),
                           static_cast<__half *>(dst), N, KG);
    }
    return check_launch("wscale relayout");
}

int launch_act_to_v1(const void *qact, const void *scale_h, int64_t M, int64_t K, void *qact_v1, void *ascales_v1, hipStream_t s) {
    const int64_t PM = ceil_div(M, 256) * 256;
    if (PM == 0) return VDMQ_OK;
    hipLaunchKernelGGL(act_to_v1_kernel, dim3(blocks_for(PM * (K / 8))), dim3(256), 0, s, static_cast<const uint32_t *>(qact),
                       static_cast<const __half *>(scale_h), M, PM, static_cast<int>(K), static_cast<int>(k_padded(K)),
                       static_cast<uint32_t *>(qact_v1), static_cast<__half *>(ascales_v1));
    return check_launch("act_to_v1_kernel");
}

int launch_act_to_native(const void *qact_v1, const void *ascales_v1, int64_t M, int64_t K, void *qact, void *scale_h,
                         hipStream_t s) {
    if (M == 0) return VDMQ_OK;
    const int Kp = static_cast<int>(k_padded(K));
    hipLaunchKernelGGL(act_to_native_kernel, dim3(blocks_for(M * (Kp / 8))), dim3(256), 0, s, static_cast<const uint32_t *>(qact_v1),
                       static_cast<const __half *>(ascales_v1), M, static_cast<int>(K), Kp, static_cast<uint32_t *>(qact),
                       static_cast<__half *>(scale_h));
    return check_launch("act_to_native_kernel");
}

}  // namespace vdmq
