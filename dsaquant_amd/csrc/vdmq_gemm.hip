// W4A4 GEMM for gfx950 (CDNA4 has no int4 MFMA).
//
//   acc[m,n] = sum_k qx[m,k] * qw[n,k]   exact int32
//   out[m,n] = fp16(float(acc) * (float(as[m]) * float(ws[n]))) (+ bias[n] in fp16)
//
// Packed int4 tiles of both operands (row-major, 64 bytes = 128 k per row and
// K step) are staged through LDS.  A lane reads 16 bytes (32 nibbles) of one
// row and widens each 32-bit word p into two MFMA operand registers
//     lo = (p << 4) & 0xF0F0F0F0   (even-k nibbles, as int8 = 16*q)
//     hi =  p       & 0xF0F0F0F0   (odd-k nibbles,  as int8 = 16*q)
// Both operands are widened the same way, so k pairs up correctly whatever
// order the MFMA consumes the bytes in, and v_mfma_i32_32x32x32_i8 accumulates
// 256 * sum(qx*qw) exactly (|16q| <= 128, K <= 65536 keeps |acc| < 2^31).
// The epilogue shifts the factor 256 out before converting to float.
//
// MFMA orientation: the A operand holds weight rows (n), the B operand token
// rows (m), so a lane's four consecutive accumulator registers are four
// consecutive n of one token: an 8-byte fp16 store.
#include "vdmq_internal.h"

namespace vdmq {
namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));

constexpr int kRowBytes = kKStep / 2; /* bytes of one operand row per K step */

// LDS byte offset of 16-byte piece `p` (0..3) of tile row `r`.  XOR-ing the
// piece index with (r/4)%4 spreads 16 consecutive rows reading the same piece
// over all 64 banks.
__device__ __forceinline__ int lds_piece_offset(int r, int p) { return r * kRowBytes + ((p ^ ((r >> 2) & 3)) << 4); }

__device__ __forceinline__ v4i widen(uint32_t p0, uint32_t p1) {
    v4i r;
    r[0] = static_cast<int>((p0 << 4) & 0xF0F0F0F0u);
    r[1] = static_cast<int>(p0 & 0xF0F0F0F0u);
    r[2] = static_cast<int>((p1 << 4) & 0xF0F0F0F0u);
    r[3] = static_cast<int>(p1 & 0xF0F0F0F0u);
    return r;
}

template <int BM, int BN, int WAVES_M, int WAVES_N>
struct GemmCfg {
    static constexpr int kThreads = WAVES_M * WAVES_N * kWaveSize;
    static constexpr int kWaveM = BM / WAVES_M;
    static constexpr int kWaveN = BN / WAVES_N;
    static constexpr int kMI = kWaveM / 32;
    static constexpr int kNI = kWaveN / 32;
    static constexpr int kStageBytes = (BM + BN) * kRowBytes;
    static constexpr int kPieces = (BM + BN) * 4; /* 16-byte pieces per stage */
    static constexpr int kPiecesPerThread = kPieces / kThreads;
    static_assert(kPieces % kThreads == 0, "stage must divide evenly over the threads");
    static_assert(kWaveM % 32 == 0 && kWaveN % 32 == 0, "wave tile is made of 32x32 MFMA tiles");
};

template <typename Cfg, int BM, int BN>
__device__ __forceinline__ void load_stage(u32x4 (&regs)[Cfg::kPiecesPerThread], const uint8_t *__restrict__ A,
                                           const uint8_t *__restrict__ W, int m0, int n0, int M, int N, int ldk, int kbyte) {
#pragma unroll
    for (int i = 0; i < Cfg::kPiecesPerThread; ++i) {
        const int q = i * Cfg::kThreads + threadIdx.x;
        const int r = q >> 2, p = q & 3;
        u32x4 v = {0u, 0u, 0u, 0u};
        if (r < BN) {
            const int n = n0 + r;
            if (n < N) v = *reinterpret_cast<const u32x4 *>(W + static_cast<int64_t>(n) * ldk + kbyte + p * 16);
        } else {
            const int m = m0 + (r - BN);
            if (m < M) v = *reinterpret_cast<const u32x4 *>(A + static_cast<int64_t>(m) * ldk + kbyte + p * 16);
        }
        regs[i] = v;
    }
}

template <typename Cfg>
__device__ __forceinline__ void store_stage(const u32x4 (&regs)[Cfg::kPiecesPerThread], uint8_t *lds) {
#pragma unroll
    for (int i = 0; i < Cfg::kPiecesPerThread; ++i) {
        const int q = i * Cfg::kThreads + threadIdx.x;
        *reinterpret_cast<u32x4 *>(lds + lds_piece_offset(q >> 2, q & 3)) = regs[i];
    }
}

// Rows 0..BN-1 of a stage are weight rows, rows BN..BN+BM-1 token rows.
template <int BM, int BN, int WAVES_M, int WAVES_N, bool ACC_OUT>
__global__ __launch_bounds__(WAVES_M *WAVES_N *kWaveSize) void gemm_w4a4_kernel(
    const uint8_t *__restrict__ A, const uint8_t *__restrict__ W, const __half *__restrict__ ascale,
    const __half *__restrict__ wscale, const __half *__restrict__ bias, void *__restrict__ out, int out_dtype,
    int32_t *__restrict__ acc_out, int M, int N, int ldk, int64_t ldo, int tiles_n) {
    using Cfg = GemmCfg<BM, BN, WAVES_M, WAVES_N>;
    __shared__ __attribute__((aligned(16))) uint8_t lds[2][Cfg::kStageBytes];

    const int tile_m = blockIdx.x / tiles_n;
    const int tile_n = blockIdx.x % tiles_n;
    const int m0 = tile_m * BM, n0 = tile_n * BN;
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int wm0 = (wave / WAVES_N) * Cfg::kWaveM; /* within the tile */
    const int wn0 = (wave % WAVES_N) * Cfg::kWaveN;
    const int l32 = lane & 31, lh = lane >> 5;

    v16i acc[Cfg::kNI][Cfg::kMI];
#pragma unroll
    for (int ni = 0; ni < Cfg::kNI; ++ni)
#pragma unroll
        for (int mi = 0; mi < Cfg::kMI; ++mi)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[ni][mi][r] = 0;

    const int ksteps = ldk / kRowBytes;
    u32x4 regs[Cfg::kPiecesPerThread];
    load_stage<Cfg, BM, BN>(regs, A, W, m0, n0, M, N, ldk, 0);
    store_stage<Cfg>(regs, lds[0]);
    __syncthreads();

    for (int kt = 0; kt < ksteps; ++kt) {
        const uint8_t *cur = lds[kt & 1];
        if (kt + 1 < ksteps) load_stage<Cfg, BM, BN>(regs, A, W, m0, n0, M, N, ldk, (kt + 1) * kRowBytes);

#pragma unroll
        for (int j = 0; j < 2; ++j) {
            u32x4 wf[Cfg::kNI], xf[Cfg::kMI];
#pragma unroll
            for (int ni = 0; ni < Cfg::kNI; ++ni)
                wf[ni] = *reinterpret_cast<const u32x4 *>(cur + lds_piece_offset(wn0 + ni * 32 + l32, 2 * j + lh));
#pragma unroll
            for (int mi = 0; mi < Cfg::kMI; ++mi)
                xf[mi] = *reinterpret_cast<const u32x4 *>(cur + lds_piece_offset(BN + wm0 + mi * 32 + l32, 2 * j + lh));
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                v4i a[Cfg::kNI], b[Cfg::kMI];
#pragma unroll
                for (int ni = 0; ni < Cfg::kNI; ++ni) a[ni] = h ? widen(wf[ni].z, wf[ni].w) : widen(wf[ni].x, wf[ni].y);
#pragma unroll
                for (int mi = 0; mi < Cfg::kMI; ++mi) b[mi] = h ? widen(xf[mi].z, xf[mi].w) : widen(xf[mi].x, xf[mi].y);
#pragma unroll
                for (int ni = 0; ni < Cfg::kNI; ++ni)
#pragma unroll
                    for (int mi = 0; mi < Cfg::kMI; ++mi)
                        acc[ni][mi] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[ni], b[mi], acc[ni][mi], 0, 0, 0);
            }
        }

        if (kt + 1 < ksteps) store_stage<Cfg>(regs, lds[(kt + 1) & 1]);
        __syncthreads();
    }

    // Epilogue.  Accumulator register r of a 32x32 tile holds
    // n = 8*(r/4) + 4*(lane/32) + r%4, m = lane%32.
#pragma unroll
    for (int mi = 0; mi < Cfg::kMI; ++mi) {
        const int m = m0 + wm0 + mi * 32 + l32;
        if (m >= M) continue;
        float as = 0.0f;
        if (!ACC_OUT) as = static_cast<float>(reinterpret_cast<const _Float16 *>(ascale)[m]);
#pragma unroll
        for (int ni = 0; ni < Cfg::kNI; ++ni) {
#pragma unroll
            for (int rg = 0; rg < 4; ++rg) {
                const int n = n0 + wn0 + ni * 32 + rg * 8 + lh * 4;
                if (n >= N) continue;
                if (ACC_OUT) {
                    v4i o;
#pragma unroll
                    for (int e = 0; e < 4; ++e) o[e] = acc[ni][mi][rg * 4 + e] >> 8;
                    *reinterpret_cast<v4i *>(acc_out + static_cast<int64_t>(m) * N + n) = o;
                } else {
                    const f16x4 ws = *reinterpret_cast<const f16x4 *>(wscale + n);
                    float v[4];
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        v[e] = static_cast<float>(acc[ni][mi][rg * 4 + e] >> 8) * (as * static_cast<float>(ws[e]));
                    if (out_dtype == VDMQ_OUT_F16) {
                        // float -> _Float16 conversions round to nearest even
                        f16x4 h = {static_cast<_Float16>(v[0]), static_cast<_Float16>(v[1]), static_cast<_Float16>(v[2]),
                                   static_cast<_Float16>(v[3])};
                        if (bias != nullptr) h += *reinterpret_cast<const f16x4 *>(bias + n); /* one fp16 add per element */
                        *reinterpret_cast<f16x4 *>(static_cast<__half *>(out) + static_cast<int64_t>(m) * ldo + n) = h;
                    } else {
                        // bf16 output (not offered by the reference): same fp32 product, the
                        // fp16-rounded bias added in fp32, one rounding to bf16.
                        uint32_t o[2];
#pragma unroll
                        for (int e2 = 0; e2 < 2; ++e2) {
                            uint32_t pk = 0;
#pragma unroll
                            for (int e = 0; e < 2; ++e) {
                                float f = v[2 * e2 + e];
                                if (bias != nullptr) f += static_cast<float>(reinterpret_cast<const _Float16 *>(bias)[n + 2 * e2 + e]);
                                uint32_t u = __float_as_uint(f);
                                u = (f != f) ? 0x7FC00000u : u + 0x7FFFu + ((u >> 16) & 1u); /* RNE */
                                pk |= (u >> 16) << (16 * e);
                            }
                            o[e2] = pk;
                        }
                        u32x2 ov = {o[0], o[1]};
                        *reinterpret_cast<u32x2 *>(static_cast<uint16_t *>(out) + static_cast<int64_t>(m) * ldo + n) = ov;
                    }
                }
            }
        }
    }
}

template <int BM, int BN, int WAVES_M, int WAVES_N>
int launch_cfg(const uint8_t *qact, const __half *ascale, const uint8_t *wq, const __half *wscale, const __half *bias, void *out,
               int out_dtype, int32_t *acc_out, int64_t M, int64_t N, int64_t K, int64_t ldo, hipStream_t s) {
    const int tiles_m = static_cast<int>(ceil_div(M, BM));
    const int tiles_n = static_cast<int>(ceil_div(N, BN));
    const int ldk = static_cast<int>(k_padded(K) / 2);
    const dim3 grid(static_cast<unsigned>(tiles_m) * tiles_n), block(WAVES_M * WAVES_N * kWaveSize);
    if (acc_out != nullptr) {
        hipLaunchKernelGGL((gemm_w4a4_kernel<BM, BN, WAVES_M, WAVES_N, true>), grid, block, 0, s, qact, wq, ascale, wscale, bias, out,
                           out_dtype, acc_out, static_cast<int>(M), static_cast<int>(N), ldk, ldo, tiles_n);
    } else {
        hipLaunchKernelGGL((gemm_w4a4_kernel<BM, BN, WAVES_M, WAVES_N, false>), grid, block, 0, s, qact, wq, ascale, wscale, bias, out,
                           out_dtype, acc_out, static_cast<int>(M), static_cast<int>(N), ldk, ldo, tiles_n);
    }
    return check_launch("gemm_w4a4_kernel");
}

}  // namespace

int launch_gemm(const uint8_t *qact, const __half *ascale, const uint8_t *wq, const __half *wscale, const __half *bias, void *out,
                int out_dtype, int32_t *acc_out, int64_t M, int64_t N, int64_t K, int64_t ldo, hipStream_t s) {
    if (M == 0 || N == 0) return VDMQ_OK;
    return launch_cfg<256, 128, 2, 2>(qact, ascale, wq, wscale, bias, out, out_dtype, acc_out, M, N, K, ldo, s);
}

}  // namespace vdmq
