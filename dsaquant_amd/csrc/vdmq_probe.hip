// Matrix-pipe ceiling probe: the two MFMA instructions of the GEMM kernels in a loop that does nothing else.
//
// Every CU runs one workgroup of eight waves (two per SIMD, as the GEMM kernels do); a wave loads two sets of
// operand registers once -- 2 weight-side and 4 token-side operands each, the GEMM's 128 x 64 wave tile -- and then
// issues the 16 MFMAs of one K step of the GEMM `iters` times onto 8 accumulator tiles, with no memory access, no
// LDS access and no barrier in the loop.  What it sustains is the rate the matrix pipes reach on this part under its
// power limit for the given operand DATA (the bits that toggle in the multipliers), which is the ceiling the GEMM
// kernels are to be read against; the published peak is the same figure at the top clock.
#include "vdmq_internal.h"

namespace vdmq {
namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v16f __attribute__((ext_vector_type(16)));

constexpr int kNI = 2, kMI = 4, kSets = 2, kWaves = 8;
constexpr int kOperandsPerWave = kSets * (kNI + kMI); /* 32 bytes per lane each */

// operands: [wave of the workgroup][operand][lane] x 32 bytes (int8: the first 16; bf6: the first 24)
template <bool BF6>
__global__ __launch_bounds__(kWaves * 64, 2) void mfma_probe_kernel(const uint32_t *__restrict__ operands, int iters, int *__restrict__ out) {
#if defined(__HIP_DEVICE_COMPILE__)
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    v8i op[kOperandsPerWave];
#pragma unroll
    for (int o = 0; o < kOperandsPerWave; ++o) {
        const uint32_t *p = operands + ((static_cast<size_t>(wave) * kOperandsPerWave + o) * 64 + lane) * 8;
#pragma unroll
        for (int r = 0; r < 8; ++r) op[o][r] = static_cast<int>(p[r]);
    }
    int result = 0;
    if constexpr (BF6) {
        v16f acc[kNI][kMI];
#pragma unroll
        for (int ni = 0; ni < kNI; ++ni)
#pragma unroll
            for (int mi = 0; mi < kMI; ++mi)
#pragma unroll
                for (int r = 0; r < 16; ++r) acc[ni][mi][r] = 0.f;
        for (int it = 0; it < iters; ++it) {
#pragma unroll
            for (int s = 0; s < kSets; ++s)
#pragma unroll
                for (int ni = 0; ni < kNI; ++ni)
#pragma unroll
                    for (int mi = 0; mi < kMI; ++mi)
                        acc[ni][mi] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(op[s * (kNI + kMI) + ni], op[s * (kNI + kMI) + kNI + mi],
                                                                                      acc[ni][mi], 3, 3, 0, 0, 0, 0);
        }
#pragma unroll
        for (int ni = 0; ni < kNI; ++ni)
#pragma unroll
            for (int mi = 0; mi < kMI; ++mi)
#pragma unroll
                for (int r = 0; r < 16; ++r) result ^= __float_as_int(acc[ni][mi][r]);
    } else {
        v16i acc[kNI][kMI];
#pragma unroll
        for (int ni = 0; ni < kNI; ++ni)
#pragma unroll
            for (int mi = 0; mi < kMI; ++mi)
#pragma unroll
                for (int r = 0; r < 16; ++r) acc[ni][mi][r] = 0;
        for (int it = 0; it < iters; ++it) {
#pragma unroll
            for (int s = 0; s < kSets; ++s)
#pragma unroll
                for (int ni = 0; ni < kNI; ++ni)
#pragma unroll
                    for (int mi = 0; mi < kMI; ++mi) {
                        const v8i a = op[s * (kNI + kMI) + ni], b = op[s * (kNI + kMI) + kNI + mi];
                        acc[ni][mi] = __builtin_amdgcn_mfma_i32_32x32x32_i8(v4i{a[0], a[1], a[2], a[3]}, v4i{b[0], b[1], b[2], b[3]}, acc[ni][mi], 0, 0, 0);
                    }
        }
#pragma unroll
        for (int ni = 0; ni < kNI; ++ni)
#pragma unroll
            for (int mi = 0; mi < kMI; ++mi)
#pragma unroll
                for (int r = 0; r < 16; ++r) result ^= acc[ni][mi][r];
    }
    out[static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x] = result;
#endif
}

}  // namespace

int64_t mfma_probe_operand_bytes() { return static_cast<int64_t>(kWaves) * kOperandsPerWave * 64 * 32; }

int launch_mfma_probe(int kind, const void *operands, int iters, int workgroups, void *out, double *ops, hipStream_t s) {
    const double macs = kind == VDMQ_PROBE_BF6 ? 32.0 * 32.0 * 64.0 : 32.0 * 32.0 * 32.0;
    *ops = 2.0 * macs * kSets * kNI * kMI * static_cast<double>(iters) * kWaves * workgroups;
    if (kind == VDMQ_PROBE_BF6)
        hipLaunchKernelGGL(mfma_probe_kernel<true>, dim3(workgroups), dim3(kWaves * 64), 0, s, static_cast<const uint32_t *>(operands), iters,
                           static_cast<int *>(out));
    else
        hipLaunchKernelGGL(mfma_probe_kernel<false>, dim3(workgroups), dim3(kWaves * 64), 0, s, static_cast<const uint32_t *>(operands), iters,
                           static_cast<int *>(out));
    return check_launch("mfma_probe_kernel");
}

}  // namespace vdmq
