// W4A4 GEMM through the bf6 (E3M2) matrix path of gfx950 -- an alternative to
// the int8 kernel of vdmq_gemm.hip, selected by the caller.
//
// v_mfma_f32_32x32x64_f8f6f4 multiplies 6-bit floats at twice the int8 rate.
// E3M2 represents q / 16 exactly for every integer q of [-8, 8] (its code is
// sign << 5 | |q|: the format's denormals and first normals), products and sums
// of such values stay exact in the fp32 accumulator while the integer sum is
// below 2^24 (K <= 65536 gives 2^22), so 256 * float(acc) is the same integer
// the int8 kernel accumulates and the epilogue that follows -- the factor 256
// folded into the channel scales, a power of two -- is bit-identical.  (The
// integers themselves are E3M2 values too; on the power-bound matrix pipes the
// small codes run 2.5 % faster on the benchmark's operands, 5 % on uniformly
// distributed int4 values, and the GEMM 1.1 %.)
//
// Operand layout ("bf6 blocks"): the MFMA takes, per 32 rows x 64 k, one 192-bit string from every lane --
// lane (r % 32) + 32 * h holds the 32 six-bit codes of k = 64 * kb + 32 * h + e (code e in bits [6e, 6e + 6)).
// In LDS such a block is [64 lanes x 16 bytes (bits 0..127)][64 lanes x 8 bytes (bits 128..191)], 1536 bytes, read
// straight into the operand registers (one 128-bit and one 64-bit read per lane, conflict-free by construction):
// no widening VALU work at all.  In memory the same strings are grouped by panels of 8 rows (bf6_piece in
// vdmq_internal.h): a panel holds its k-blocks one after the other, 384 bytes each, so the activation quantizer's
// eight-row workgroups write one contiguous stream per panel (measured 9 % faster at K = 13824 than writing
// 128-byte pieces into 1536-byte blocks) and the direct-to-LDS loads still fetch whole 128-byte lines, each lane
// from its own address.  Rows are padded to 32 (zero codes), K to 128.
#include <type_traits>

#include "vdmq_bf6_tilemap.h"
#include "vdmq_internal.h"

namespace vdmq {
namespace {

typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v4i __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));

#define VDMQ_GLOBAL_PTR(p) ((const __attribute__((address_space(1))) void *)(p))
#define VDMQ_LDS_PTR(p) ((__attribute__((address_space(3))) void *)(p))

[[maybe_unused]] constexpr int waitcnt_imm(int vm, int lgkm) { return (vm & 15) | ((vm >> 4) << 14) | (7 << 4) | ((lgkm & 15) << 8); }

[[maybe_unused]] __device__ __forceinline__ void lds_barrier() {
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
}

constexpr int kBlkBytes = 1536;                 /* 32 rows x 64 k */
[[maybe_unused]] constexpr int kBlkPlaneB = 1024;                /* offset of the 8-byte plane */
constexpr int KS = 128;                         /* K step: two k-blocks per stage */
constexpr int kRbStage = (KS / 64) * kBlkBytes; /* bytes of one row-block per stage */
constexpr int kXcds = kBf6Xcds;
// The operand blocks hold q / 16, so an accumulator holds the integer sum / 256 (as exact as the sum itself: a power
// of two); the factor goes into the channel scales of the epilogue.
[[maybe_unused]] constexpr float kBf6AccScale = 256.0f;
// per wave, beside the stage ring: the fp16 token scales of its 128 rows, the channel scales and the bias of its 64
// columns, fetched when the tile starts so that the epilogue does not wait for them
[[maybe_unused]] constexpr int kSideAs = 0, kSideWs = 256, kSideBias = 384;
constexpr int kSideBytes = 512;
// the tile-walking kernel's list of its tiles, behind the waves' side vectors: (tile_m, tile_n) per round
constexpr int kTileTableEntries = 1024, kTileTableBytes = kTileTableEntries * 8;

// Tile configuration.  BM token rows x BN weight rows per workgroup, WAVES_M x WAVES_N waves (a wave owns
// 128 x 64 or 64 x 64: 4 x 2 or 2 x 2 MFMA tiles), STAGES ring slots of (BM + BN) / 32 row-blocks, OCC workgroups
// per CU.  Two configurations are instantiated.  Big: one workgroup of eight waves owns the CU, the fewest operand
// bytes per MAC.  (128 x 256 tiles with two workgroups of four waves per CU, so that one's prologue and epilogue run
// under the other's K loop, measured 2...10 % slower on every shape down to K = 1536, with and without a start
// offset between the two.)  Small: 128 x 128 tiles, two workgroups of four waves per CU, for problems that cannot
// give every CU a big tile; only the one-workgroup-per-tile kernel has it.
template <int BM_, int BN_, int WAVES_M_, int WAVES_N_, int STAGES_, int OCC_>
struct Bf6Cfg {
    static constexpr int BM = BM_, BN = BN_, kWavesM = WAVES_M_, kWavesN = WAVES_N_, kWaves = WAVES_M_ * WAVES_N_, S = STAGES_, kOcc = OCC_;
    static constexpr int MI = BM / 32 / kWavesM, NI = BN / 32 / kWavesN; /* 32-row blocks per wave: token, weight */
    static constexpr int kStageBytes = (BM + BN) / 32 * kRbStage;
    static constexpr int kLoads = kStageBytes / 1024 / kWaves;
    static constexpr int kRingBytes = S * kStageBytes;
    static constexpr int kTableOffset = kRingBytes + kWaves * kSideBytes;
    static constexpr int kLdsBytes = kTableOffset + kTileTableBytes; /* stage ring + the waves' scale and bias vectors + tile list */
    static constexpr int kLdsBytesOneTile = kTableOffset;            /* the one-workgroup-per-tile kernel keeps no list */
    static constexpr int kWaveN = NI * 32;
    static constexpr int kStageRowBytes = kWaveN * 2 + 16; /* epilogue staging: fp16 strip rows padded by 16 bytes */
    static constexpr int kStagingBytes = 32 * kStageRowBytes;
    static constexpr int kPiecesPerRow = kWaveN / 8;
    static constexpr int kPerLog2 = BM == 256 ? 5 : 6; /* tiles per super-tile: what an XCD's 32 CUs hold at once */
    static_assert((MI == 4 || MI == 2) && NI == 2, "the schedule below is written for 128 x 64 and 64 x 64 wave tiles");
    static_assert(kStagingBytes * kWaves <= kRingBytes, "epilogue staging reuses the stage ring");
    static_assert(kStageBytes % (1024 * kWaves) == 0, "stage splits evenly over the waves");
    static_assert(kLoads * (S - 1) < 64, "vmcnt is a 6-bit counter");
    static_assert((kOcc == 1 ? kLdsBytes : kLdsBytesOneTile) * kOcc <= 160 * 1024, "the CU's LDS holds OCC workgroups");
};
using Bf6Big = Bf6Cfg<256, 256, 2, 4, 3, 1>;
using Bf6Small = Bf6Cfg<128, 128, 2, 2, 3, 2>;

// workgroup b runs on XCD b % 8; each XCD walks super-tiles (vdmq_bf6_tilemap.h)
[[maybe_unused]] __device__ __forceinline__ bool map_tile(const Bf6TileMap &tm, int bid, int &tile_m, int &tile_n) {
    const int xcd = bid % kXcds, slot = bid / kXcds;
    const int st = bf6_tilemap_super(tm, xcd, slot >> tm.per_log2);
    return st >= 0 && bf6_tilemap_locate(tm, st, slot & ((1 << tm.per_log2) - 1), tile_m, tile_n);
}

[[maybe_unused]] __device__ __forceinline__ v8i ld_frag(const uint8_t *p, uint32_t la, uint32_t lb) {
    const u32x4 a = *reinterpret_cast<const u32x4 *>(p + la);
    const u32x2 b = *reinterpret_cast<const u32x2 *>(p + lb);
    v8i r = {(int)a.x, (int)a.y, (int)a.z, (int)a.w, (int)b.x, (int)b.y, 0, 0}; /* the MFMA reads six registers */
    return r;
}

#if defined(__HIP_DEVICE_COMPILE__) /* (the host pass does not know the buffer builtins) */
// The K loop of one tile, shared by the two kernels.
//
// One K step = two k-blocks of eight MFMAs each (the wave's 2 x 4 MFMA tiles).  Fragment f of a k-block (0: weight
// rows 0-31, 1...4: the four token row-blocks, 5: weight rows 32-63 -- the order in which the MFMAs first need them)
// is read from LDS behind the f-th MFMA of the k-block before it.  The six global -> LDS loads of a stage go out
// three per k-block, behind every other MFMA (kLoadSlots*): loads 3...5 of stage kt + 2 in the first k-block of step kt, loads
// 0...2 of stage kt + 3 in its second one, each into a ring slot whose last reader has passed a barrier.  That way
// the CU's eight waves hand the texture path one load every few cycles; issued together, 48 at a time, they queue
// up in front of it, and a wave that cannot issue its load cannot issue the MFMAs behind it either (all six behind
// the k-block's last MFMAs: 6.5 % slower on the 14B shapes).  Direct-to-LDS loads and LDS reads keep their program
// order -- the compiler sees one LDS and orders every such pair -- so the order written here, pinned per MFMA by
// sched_barrier, is the order of the instruction stream; scheduling hints alone cannot move a load in front of an
// LDS read that precedes it in the source.
//
// On entry stages 0, 1 and 2 of the tile are requested (0 and 1 landed and published), `cur` is the ring slot of
// stage 0 and wfa / xfa hold its first k-block's fragments.  `ksteps` K steps are worked; stage t lies at K step
// ksteps - 1 - t of the operands if `k_reverse`, else at t.
template <class Cfg>
struct Bf6KLoop {
    static constexpr int NI = Cfg::NI, MI = Cfg::MI, S = Cfg::S, kLoads = Cfg::kLoads, kWaves = Cfg::kWaves, BN = Cfg::BN;
    static_assert(NI == 2 && (MI == 4 || MI == 2) && kLoads == 6 && S == 3, "the schedule is written for these shapes");
    // MFMAs of a k-block (bit i = behind the i-th) that are followed by a load: behind the 2nd, 4th and 6th in the first
    // k-block, the 3rd, 5th and 7th in the second.  Measured against other triples: a load behind a k-block's first
    // MFMA (right after the barrier, or the loop's head) costs 2 %, the rest lie within 1 %.
    // (64 x 64 wave tiles have four MFMAs per k-block: behind the 2nd, 3rd and 4th)
    static constexpr unsigned kLoadSlotsB = MI == 4 ? 0x2A : 0xE, kLoadSlotsA = MI == 4 ? 0x54 : 0xE;
    uint8_t *lds;
    const __amdgpu_buffer_rsrc_t (&src)[kLoads];
    const uint32_t (&lane_off)[kLoads];
    int wave, wn, wm;
    uint32_t la, lb;
    int ksteps;
    bool k_reverse;

    __device__ __forceinline__ v8i frag_at(const uint8_t *stage, int f, int kb) const {
        const int rb = f == 0 ? wn * NI : (f == NI + MI - 1 ? wn * NI + 1 : BN / 32 + wm * MI + f - 1);
        return ld_frag(stage + (rb * 2 + kb) * kBlkBytes, la, lb);
    }
    static __device__ __forceinline__ void put(v8i (&wf)[NI], v8i (&xf)[MI], int f, const v8i &v) {
        if (f == 0) wf[0] = v;
        else if (f == NI + MI - 1) wf[1] = v;
        else xf[f - 1] = v;
    }
    __device__ __forceinline__ void load_one(int i, int stage_no, int slot) const {
        const int kpos = k_reverse ? ksteps - 1 - stage_no : stage_no;
        __builtin_amdgcn_raw_ptr_buffer_load_lds(src[i], VDMQ_LDS_PTR(lds + slot * Cfg::kStageBytes + (i * kWaves + wave) * 1024), 16, lane_off[i],
                                                 kpos * (KS / 64) * kBf6PanelKb, 0, 0);
    }
    // LOAD_B / LOAD_A: this step issues the second half of stage kt + 2 / the first half of stage kt + 3; READ_NEXT: a
    // step follows; YOUNGER: stage kt + 2 exists, i.e. six loads may stay in flight across the barrier (-1: look at kt);
    // FIRST: the tile's first step, whose first eight MFMAs start the accumulators from the constant zero, so that
    // nobody clears 128 registers per wave between two tiles (the Wan-1.3B block's GEMMs, 12-step tiles: +2.4 %)
    template <bool LOAD_B, bool LOAD_A, bool READ_NEXT, int YOUNGER, bool FIRST = false>
    __device__ __forceinline__ void step(int kt, int &cur, v16f (&acc)[NI][MI], v8i (&wfa)[NI], v8i (&xfa)[MI], v8i (&wfb)[NI],
                                         v8i (&xfb)[MI]) const {
        const uint8_t *stage = lds + cur * Cfg::kStageBytes;
        const int nxt = cur + 1 == S ? 0 : cur + 1, prv = cur == 0 ? S - 1 : cur - 1;
#pragma unroll
        for (int i = 0; i < NI * MI; ++i) {
            const v16f zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
            acc[i / MI][i % MI] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(wfa[i / MI], xfa[i % MI], FIRST ? zero : acc[i / MI][i % MI], 3, 3, 0, 0,
                                                                                 0, 0); /* bf6 x bf6, no scaling */
            if (i < NI + MI) put(wfb, xfb, i, frag_at(stage, i, 1));
            if (LOAD_B && ((kLoadSlotsB >> i) & 1)) load_one(kLoads / 2 + __builtin_popcount(kLoadSlotsB & ((1 << i) - 1)), kt + 2, prv);
            __builtin_amdgcn_sched_barrier(0);
        }
        // one barrier per step: behind it stage kt + 1 is complete for every wave (the stage after it may still be on
        // its way: six loads), and nobody reads slot `cur` any more
        if (YOUNGER > 0 || (YOUNGER < 0 && kt + 2 < ksteps))
            __builtin_amdgcn_s_waitcnt(waitcnt_imm(kLoads, 0));
        else
            __builtin_amdgcn_s_waitcnt(waitcnt_imm(0, 0));
        lds_barrier();
#pragma unroll
        for (int i = 0; i < NI * MI; ++i) {
            acc[i / MI][i % MI] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(wfb[i / MI], xfb[i % MI], acc[i / MI][i % MI], 3, 3, 0, 0, 0, 0);
            if (READ_NEXT && i < NI + MI) put(wfa, xfa, i, frag_at(lds + nxt * Cfg::kStageBytes, i, 0));
            if (LOAD_A && ((kLoadSlotsA >> i) & 1)) load_one(__builtin_popcount(kLoadSlotsA & ((1 << i) - 1)), kt + 3, cur);
            __builtin_amdgcn_sched_barrier(0);
        }
        cur = nxt;
    }
    // (The kernel that walks tiles has a tile's first two stages landed when it gets here, so its step 0 could skip
    // the wait -- which, loads and stores sharing one counter, also waits for the output stores of the tile before --
    // but a build that does measured the same time to 0.1 % on the 14B and 1.3B blocks: one form for both kernels.)
    __device__ __forceinline__ void run(int &cur, v16f (&acc)[NI][MI], v8i (&wfa)[NI], v8i (&xfa)[MI], v8i (&wfb)[NI], v8i (&xfb)[MI]) const {
        int kt = 0;
        if (ksteps > S) {
            step<false, true, true, 1, true>(0, cur, acc, wfa, xfa, wfb, xfb);
            for (kt = 1; kt + S < ksteps; ++kt) step<true, true, true, 1>(kt, cur, acc, wfa, xfa, wfb, xfb);
            step<true, false, true, 1>(kt, cur, acc, wfa, xfa, wfb, xfb);
            ++kt;
        } else { /* (at most three K steps: cleared the plain way; a second first-step variant here and the register
                    allocator no longer finds one home for the accumulators of both paths) */
#pragma unroll
            for (int ni = 0; ni < NI; ++ni)
#pragma unroll
                for (int mi = 0; mi < MI; ++mi)
#pragma unroll
                    for (int r = 0; r < 16; ++r) acc[ni][mi][r] = 0.f;
        }
        for (; kt + 1 < ksteps; ++kt) step<false, false, true, -1>(kt, cur, acc, wfa, xfa, wfb, xfb);
        step<false, false, false, 0>(kt, cur, acc, wfa, xfa, wfb, xfb);
    }
};

// fp16 epilogue of one wave's 128 x 64 corner of a tile, as in the int8 kernel:
// out = fp16(float(acc) * (float(as) * float(ws))) (+ bias in fp16) [then residual + y * gate]; one 32-row strip at
// a time is transposed through the wave's staging area so that rows leave as whole 128-byte lines.  `side` holds the
// wave's token scales, channel scales and bias; (m0, n0) is the corner's first output element.  `before_first_store`
// runs once, after the first strip has been converted and staged.  BF16: the same fp32 product, the fp16 bias added in
// fp32 and one rounding (to nearest even) to bf16, as the int8 kernel writes a bf16 output; no tail.
template <class Cfg, bool STREAM_OUT, bool TAIL, bool BF16, class Hook>
__device__ __forceinline__ void bf6_epilogue(const v16f (&acc)[Cfg::NI][Cfg::MI], const uint8_t *side, uint8_t *stg, int lane, int m0, int n0,
                                             __half *out, int64_t ldo, int M, int N, const GemmTail &tail, Hook &&before_first_store) {
    constexpr int MI = Cfg::MI, NI = Cfg::NI, PR = Cfg::kPiecesPerRow, RS = Cfg::kStageRowBytes;
    const int l32 = lane & 31, lh = lane >> 5;
    float wsf[NI][4][4];
#pragma unroll
    for (int ni = 0; ni < NI; ++ni)
#pragma unroll
        for (int rg = 0; rg < 4; ++rg) {
            const f16x4 w4 = *reinterpret_cast<const f16x4 *>(side + kSideWs + (ni * 32 + rg * 8 + lh * 4) * 2);
#pragma unroll
            for (int e = 0; e < 4; ++e) wsf[ni][rg][e] = static_cast<float>(w4[e]) * kBf6AccScale; /* exact: a power of two */
        }
    const int ncol = n0 + (lane % PR) * 8;
    const f16x8 bv = *reinterpret_cast<const f16x8 *>(side + kSideBias + (lane % PR) * 16); /* -0 without a bias */
    // The stores are buffer stores: the wave's corner of the output is the resource, whose size ends with the last
    // row below M, so rows beyond are dropped by the range check instead of being predicated.  The check looks at the
    // vector offset only (a scalar offset is added after it), so the row goes into the vector offset: one addition
    // per store where a 64-bit address takes a multiplication and several additions.
    const int wave_rows = min(M - m0, MI * 32);
    const int part = tail.split_cols != 0 ? n0 / tail.split_cols : 0; /* the wave's 64 columns lie inside one part */
    const __amdgpu_buffer_rsrc_t out_rsrc = __builtin_amdgcn_make_buffer_rsrc(
        out + part * tail.part_stride + static_cast<int64_t>(m0) * ldo + (n0 - part * tail.split_cols), 0, wave_rows * static_cast<int>(ldo) * 2,
        0x00020000);
    const int out_voff = ((lane / PR) * static_cast<int>(ldo) + (lane % PR) * 8) * 2;
    // Row of the gate vectors for output row m = m / rows_per_gate, without a division per element: one vector per
    // token is the row itself, and with at least as many rows per vector as the wave owns the wave's rows meet at
    // most one boundary, found by comparing with the first row's remainder.
    const int gate_rows = TAIL ? tail.rows_per_gate : 1;
    const int gate_first = __builtin_amdgcn_readfirstlane(m0 / gate_rows), gate_rem = m0 - gate_first * gate_rows;
    auto gate_row = [&](int mrow) -> int64_t {
        if (gate_rows == 1) return mrow;
        if (gate_rows >= MI * 32) return gate_first + (gate_rem + (mrow - m0) >= gate_rows ? 1 : 0);
        return mrow / gate_rows;
    };
#pragma unroll
    for (int mi = 0; mi < MI; ++mi) {
        const float as = static_cast<float>(*reinterpret_cast<const _Float16 *>(side + kSideAs + (mi * 32 + l32) * 2));
        // gate and residual pieces of this strip, requested before the strip is converted and staged
        f16x8 gv[PR / 2], rv[PR / 2];
#pragma unroll
        for (int it = 0; TAIL && it < PR / 2; ++it) {
            const int mrow = m0 + mi * 32 + it * (64 / PR) + lane / PR;
            const bool live = mrow < M && ncol < N;
            if (tail.gate != nullptr && live)
                gv[it] = *reinterpret_cast<const f16x8 *>(tail.gate + gate_row(mrow) * tail.ldg + ncol);
            if (tail.residual != nullptr && live)
                rv[it] = *reinterpret_cast<const f16x8 *>(tail.residual + static_cast<int64_t>(mrow) * tail.ldr + ncol);
        }
#pragma unroll
        for (int ni = 0; ni < NI; ++ni)
#pragma unroll
            for (int rg = 0; rg < 4; ++rg) {
                if (BF16) {
                    const f16x4 b4 = *reinterpret_cast<const f16x4 *>(side + kSideBias + (ni * 32 + rg * 8 + lh * 4) * 2);
                    uint32_t o[2] = {0, 0};
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const float f = acc[ni][mi][rg * 4 + e] * (as * wsf[ni][rg][e]) + static_cast<float>(b4[e]); /* -0: no bias */
                        uint32_t u = __float_as_uint(f);
                        u = (f != f) ? 0x7FC00000u : u + 0x7FFFu + ((u >> 16) & 1u);
                        o[e / 2] |= (u >> 16) << (16 * (e % 2));
                    }
                    *reinterpret_cast<u32x2 *>(stg + l32 * RS + (ni * 32 + rg * 8 + lh * 4) * 2) = u32x2{o[0], o[1]};
                } else {
                    f16x4 h;
#pragma unroll
                    for (int e = 0; e < 4; ++e) h[e] = static_cast<_Float16>(acc[ni][mi][rg * 4 + e] * (as * wsf[ni][rg][e]));
                    *reinterpret_cast<f16x4 *>(stg + l32 * RS + (ni * 32 + rg * 8 + lh * 4) * 2) = h;
                }
            }
        if (mi == 0) before_first_store();
#pragma unroll
        for (int it = 0; it < PR / 2; ++it) {
            const int row = it * (64 / PR) + lane / PR;
            f16x8 hv = *reinterpret_cast<const f16x8 *>(stg + row * RS + (lane % PR) * 16);
            if (!BF16) hv += bv;
            const int mrow = m0 + mi * 32 + row;
            if (TAIL && tail.gate != nullptr && mrow < M) hv *= gv[it];
            if (TAIL && tail.residual != nullptr && mrow < M) hv = rv[it] + hv;
            __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, hv), out_rsrc,
                                                   out_voff + (mi * 32 + it * (64 / PR)) * static_cast<int>(ldo) * 2, 0,
                                                   STREAM_OUT ? 2 /* nt */ : 0);
        }
    }
}
#endif

// Timing aid, off in the shipped library: a build with -DVDMQ_DBG_TIMELINE stamps the 100 MHz clock at five points of
// every tile of the tile-walking kernel (thread 0 of each workgroup, first 64 tiles) into a device array that
// vdmq_debug_timeline copies out: K loop, next tile's requests, epilogue, wait at the barrier (and the kernel's entry).
#ifdef VDMQ_DBG_TIMELINE
__device__ uint64_t g_timeline[256][64][6];
#define VDMQ_STAMP(tile, i) do { if (threadIdx.x == 0 && (tile) < 64) g_timeline[blockIdx.x][tile][i] = wall_clock64(); } while (0)
#else
#define VDMQ_STAMP(tile, i) do { } while (0)
#endif

// OUT_MODE: 0 = scaled fp16 output, 1 = the same with non-temporal stores, 2 = raw accumulators as int32,
// 3 / 4 = 0 / 1 followed by the gated residual update out = residual + y * gate (see vdmq_gemm.hip), 5 / 6 = 0 / 1 with
// a bf16 output
template <class Cfg, int OUT_MODE>
__global__ __launch_bounds__(Cfg::kWaves * 64, (Cfg::kWaves * Cfg::kOcc + 3) / 4) void gemm_bf6_kernel(const uint8_t *__restrict__ X, const uint8_t *__restrict__ W,
                                                                         const __half *__restrict__ ascale,
                                                                         const __half *__restrict__ wscale,
                                                                         const __half *__restrict__ bias, __half *out,
                                                                         int32_t *__restrict__ acc_out, int M, int N, int kblocks,
                                                                         int64_t ldo, Bf6TileMap tmap, GemmTail tail) {
#if defined(__HIP_DEVICE_COMPILE__) /* the host pass needs the kernel's stub only; it does not know the buffer builtins */
    constexpr bool ACC_OUT = OUT_MODE == 2, STREAM_OUT = OUT_MODE == 1 || OUT_MODE == 4 || OUT_MODE == 6;
    constexpr bool TAIL = OUT_MODE == 3 || OUT_MODE == 4, BF16 = OUT_MODE >= 5;
    constexpr int BM = Cfg::BM, BN = Cfg::BN, S = Cfg::S, MI = Cfg::MI, NI = Cfg::NI, kWaves = Cfg::kWaves, kWavesN = Cfg::kWavesN;
    constexpr int kLoads = Cfg::kLoads, kStageBytes = Cfg::kStageBytes;
    constexpr int kStagingBytes = Cfg::kStagingBytes;
    extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];
    int tile_m, tile_n;
    if (!map_tile(tmap, blockIdx.x, tile_m, tile_n)) return;
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int wn = wave % kWavesN, wm = wave / kWavesN;
    const int last_rb_m = (M + 31) / 32 - 1, last_rb_n = N / 32 - 1;
    // global -> LDS: a stage is (BN + BM) / 32 row-blocks x 3 KiB, weights first; this wave's i-th instruction fills
    // KiB (i * kWaves + wave) of it, 16 bytes per lane.  In LDS a row-block's two k-blocks lie as the MFMA reads them,
    // [64 lanes x 16 B][64 lanes x 8 B] each; in memory the operand is stored by panels of 8 rows (bf6_piece below), so
    // every lane finds its 16 bytes -- one lane's 16-byte part or two neighbouring rows' 8-byte parts -- on its own.
    // The source of a load is a base the whole wave shares (the row-block's first panel) plus a scalar offset that
    // advances with K plus a 32-bit offset per lane that never changes -- a buffer load's three address parts, so the
    // K loop spends no vector instruction on addresses (global_load_lds wants a 64-bit address per lane).
    __amdgpu_buffer_rsrc_t src[kLoads];
    uint32_t lane_off[kLoads];
#pragma unroll
    for (int i = 0; i < kLoads; ++i) {
        const int idx = i * kWaves + wave, q = idx / 3;
        const int off = (idx % 3) * 1024 + lane * 16;    /* byte in the row-block's 3072-byte LDS image */
        const int kb = off >= kBlkBytes ? 1 : 0, in_blk = off - kb * kBlkBytes;
        const bool part_b = in_blk >= kBlkPlaneB;
        const int l = part_b ? (in_blk - kBlkPlaneB) / 8 : in_blk / 16; /* lane of the MFMA operand: row % 32 + 32 * h */
        const int64_t rb = q < BN / 32 ? min(tile_n * (BN / 32) + q, last_rb_n) : min(tile_m * (BM / 32) + q - BN / 32, last_rb_m);
        // rows past M or N re-read the last row-block and are never stored; the range covers the row-block's four panels
        src[i] = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t *>((q < BN / 32 ? W : X) + bf6_piece(rb * 32, 0, 0, false, kblocks)), 0,
                                                   4 * kblocks * kBf6PanelKb, 0x00020000 /* raw buffer of dwords */);
        lane_off[i] = static_cast<uint32_t>(bf6_piece(l & 31, kb, l >> 5, part_b, kblocks));
    }
    // every other super-tile of an XCD's run walks K backwards (sums of integers: any order gives the same result)
    const bool k_reverse = tmap.contig && (((blockIdx.x / kXcds) >> tmap.per_log2) & 1) != 0;
    const int ksteps_all = kblocks / (KS / 64);
    auto issue = [&](int kt, int slot) __attribute__((always_inline)) {
        const int kpos = k_reverse ? ksteps_all - 1 - kt : kt;
#pragma unroll
        for (int i = 0; i < kLoads; ++i)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(src[i], VDMQ_LDS_PTR(lds + slot * kStageBytes + (i * kWaves + wave) * 1024), 16,
                                                     lane_off[i], kpos * (KS / 64) * kBf6PanelKb, 0, 0);
    };
    const uint32_t la = lane * 16, lb = kBlkPlaneB + lane * 8;
    auto read = [&](v8i (&wf)[NI], v8i (&xf)[MI], const uint8_t *stage, int kb) __attribute__((always_inline)) {
#pragma unroll
        for (int ni = 0; ni < NI; ++ni) wf[ni] = ld_frag(stage + ((wn * NI + ni) * 2 + kb) * kBlkBytes, la, lb);
#pragma unroll
        for (int mi = 0; mi < MI; ++mi) xf[mi] = ld_frag(stage + ((BN / 32 + wm * MI + mi) * 2 + kb) * kBlkBytes, la, lb);
    };
    v16f acc[NI][MI]; /* (started from zero by the K loop's first MFMAs) */
    // weight rows are the A operand, token rows the B operand: accumulator register r of a 32 x 32
    // tile holds n = 8 * (r / 4) + 4 * (lane / 32) + r % 4, m = lane % 32
    const int ksteps = kblocks / (KS / 64);
    const int m0 = tile_m * BM, n0 = tile_n * BN, wm0 = wm * MI * 32, wn0 = wn * NI * 32;
    uint8_t *side = lds + Cfg::kRingBytes + wave * kSideBytes;
    // (no bias: -0, the one fp16 value whose addition changes no bit of any output)
    _Float16 side_as[2] = {0, 0}, side_ws = 0, side_bias = static_cast<_Float16>(-0.0f);
    if (!ACC_OUT) { /* older than the stage loads below: complete before the first of those is waited for */
        const _Float16 *as_p = reinterpret_cast<const _Float16 *>(ascale);
        side_as[0] = as_p[min(m0 + wm0 + lane, M - 1)];
        side_as[1] = as_p[min(m0 + wm0 + 64 + lane, M - 1)];
        side_ws = reinterpret_cast<const _Float16 *>(wscale)[min(n0 + wn0 + lane, N - 1)];
        if (bias != nullptr) side_bias = reinterpret_cast<const _Float16 *>(bias)[min(n0 + wn0 + lane, N - 1)];
    }
#pragma unroll
    for (int s = 0; s < S; ++s)
        if (s < ksteps) issue(s, s);
    if (ksteps >= S)
        __builtin_amdgcn_s_waitcnt(waitcnt_imm(kLoads * (S - 1), 15));
    else
        __builtin_amdgcn_s_waitcnt(waitcnt_imm(0, 15));
    lds_barrier();
    if (!ACC_OUT) { /* wave-private: the epilogue's reads follow these writes in the wave's own LDS queue */
        *reinterpret_cast<_Float16 *>(side + kSideAs + lane * 2) = side_as[0];
        *reinterpret_cast<_Float16 *>(side + kSideAs + 128 + lane * 2) = side_as[1];
        *reinterpret_cast<_Float16 *>(side + kSideWs + lane * 2) = side_ws;
        *reinterpret_cast<_Float16 *>(side + kSideBias + lane * 2) = side_bias;
    }
    v8i wfa[NI], xfa[MI], wfb[NI], xfb[MI];
    read(wfa, xfa, lds, 0);
    int cur = 0;
    const Bf6KLoop<Cfg> k_loop{lds, src, lane_off, wave, wn, wm, la, lb, ksteps, k_reverse};
    k_loop.run(cur, acc, wfa, xfa, wfb, xfb);

    const int l32 = lane & 31, lh = lane >> 5;
    if (ACC_OUT) {
#pragma unroll
        for (int mi = 0; mi < MI; ++mi) {
            const int m = m0 + wm0 + mi * 32 + l32;
            if (m >= M) continue;
#pragma unroll
            for (int ni = 0; ni < NI; ++ni)
#pragma unroll
                for (int rg = 0; rg < 4; ++rg) {
                    const int n = n0 + wn0 + ni * 32 + rg * 8 + lh * 4;
                    if (n >= N) continue;
                    v4i o;
#pragma unroll
                    for (int e = 0; e < 4; ++e) o[e] = static_cast<int>(acc[ni][mi][rg * 4 + e] * kBf6AccScale);
                    *reinterpret_cast<v4i *>(acc_out + static_cast<int64_t>(m) * N + n) = o;
                }
        }
        return;
    }
    if (n0 + wn0 >= N || m0 + wm0 >= M) return; /* nothing to store: the same for the whole wave */
    bf6_epilogue<Cfg, STREAM_OUT, TAIL, BF16>(acc, side, lds + wave * kStagingBytes, lane, m0 + wm0, n0 + wn0, out, ldo, M, N, tail, [] {});
#endif
}

// The same GEMM as a persistent kernel: one workgroup per CU position (XCD x, place j of a super-tile) walks that
// place of every super-tile of its XCD.  While a tile's epilogue converts and stores, the first two K steps of the
// next tile are already on their way into the two ring slots the epilogue's staging does not use; nothing is
// dispatched, and no kernel argument re-read, between tiles.
template <class Cfg, int OUT_MODE>
__global__ __launch_bounds__(Cfg::kWaves * 64, (Cfg::kWaves * Cfg::kOcc + 3) / 4) void gemm_bf6_persistent_kernel(
    const uint8_t *__restrict__ X, const uint8_t *__restrict__ W, const __half *__restrict__ ascale, const __half *__restrict__ wscale,
    const __half *__restrict__ bias, __half *out, int M, int N, int kblocks, int64_t ldo, Bf6TileMap tmap, GemmTail tail) {
#if defined(__HIP_DEVICE_COMPILE__)
    constexpr bool STREAM_OUT = OUT_MODE == 1 || OUT_MODE == 4 || OUT_MODE == 6, TAIL = OUT_MODE == 3 || OUT_MODE == 4, BF16 = OUT_MODE >= 5;
    constexpr int BM = Cfg::BM, BN = Cfg::BN, S = Cfg::S, MI = Cfg::MI, NI = Cfg::NI, kWaves = Cfg::kWaves, kWavesN = Cfg::kWavesN;
    constexpr int kLoads = Cfg::kLoads, kStageBytes = Cfg::kStageBytes;
    static_assert(S == 3, "the prefetch under the epilogue uses ring slots 1 and 2");
    extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];
    VDMQ_STAMP(0, 5); /* kernel entry */
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int wn = wave % kWavesN, wm = wave / kWavesN;
    const int wm0 = wm * MI * 32, wn0 = wn * NI * 32;
    const int last_rb_m = (M + 31) / 32 - 1, last_rb_n = N / 32 - 1;
    const int ksteps = kblocks / (KS / 64);
    const int xcd = blockIdx.x % kXcds, place = blockIdx.x / kXcds; /* gridDim.x = kXcds << per_log2 */
    // the seq-th super-tile of this XCD, and this workgroup's tile in it (false: none left; a super-tile at a ragged
    // edge may have no tile at this place: tile_m = -1)
    auto locate = [&](int seq, int &tile_m, int &tile_n) -> bool {
        const int st = bf6_tilemap_super(tmap, xcd, seq);
        if (st < 0) return false;
        if (!bf6_tilemap_locate(tmap, st, place, tile_m, tile_n)) tile_m = -1;
        return true;
    };
    // The workgroup's tiles, round by round, are worked out once, a round per thread, and kept in LDS: between two
    // tiles -- matrix pipes idle, every wave running the same scalar code -- finding the next tile is then one LDS
    // read instead of the map's divisions and case distinctions (150 scalar instructions per wave and tile).  Entry:
    // tile_m (-1: no tile at this place in that round, -2: no such round), tile_n.  Launches with more rounds than the
    // table holds work the map out tile by tile as before.  The table is filled while the first tile's loads are on
    // their way (below), for the rounds this XCD has and the entry behind them.
    int2 *tile_table = reinterpret_cast<int2 *>(lds + Cfg::kTableOffset);
    const int my_rounds = tmap.contig ? tmap.start[xcd + 1] - tmap.start[xcd] : (tmap.total_super + kXcds - 1) / kXcds;
    const bool tabled = my_rounds < kTileTableEntries;
    auto fill_tile_table = [&] {
        for (int e = threadIdx.x; tabled && e <= my_rounds; e += Cfg::kWaves * 64) {
            int2 ent = {-2, 0};
            if (!locate(e, ent.x, ent.y)) ent.x = -2;
            tile_table[e] = ent;
        }
    };
    // Advances seq to the next existing tile; `skipped` counts the super-tiles passed on the way in which this place
    // has no tile (a ragged edge).
    auto next_tile = [&](int &seq, int &tile_m, int &tile_n, int &skipped) -> bool {
        skipped = 0;
        for (;;) {
            ++seq;
            if (tabled) {
                const int2 ent = tile_table[seq]; /* (seq stays below the table's size: the entry behind the last round says -2) */
                tile_m = __builtin_amdgcn_readfirstlane(ent.x);
                tile_n = __builtin_amdgcn_readfirstlane(ent.y);
                if (tile_m == -2) return false;
            } else if (!locate(seq, tile_m, tile_n)) {
                return false;
            }
            if (tile_m >= 0) return true;
            ++skipped;
        }
    };
    uint32_t lane_off[kLoads];
#pragma unroll
    for (int i = 0; i < kLoads; ++i) {
        const int off = ((i * kWaves + wave) % 3) * 1024 + lane * 16;
        const int kb = off >= kBlkBytes ? 1 : 0, in_blk = off - kb * kBlkBytes;
        const bool part_b = in_blk >= kBlkPlaneB;
        const int l = part_b ? (in_blk - kBlkPlaneB) / 8 : in_blk / 16;
        lane_off[i] = static_cast<uint32_t>(bf6_piece(l & 31, kb, l >> 5, part_b, kblocks));
    }
    auto sources = [&](__amdgpu_buffer_rsrc_t (&src)[kLoads], int tile_m, int tile_n) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < kLoads; ++i) {
            const int q = (i * kWaves + wave) / 3;
            const int64_t rb = q < BN / 32 ? min(tile_n * (BN / 32) + q, last_rb_n) : min(tile_m * (BM / 32) + q - BN / 32, last_rb_m);
            src[i] = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t *>((q < BN / 32 ? W : X) + bf6_piece(rb * 32, 0, 0, false, kblocks)), 0,
                                                       4 * kblocks * kBf6PanelKb, 0x00020000);
        }
    };
    auto issue = [&](const __amdgpu_buffer_rsrc_t (&src)[kLoads], bool k_reverse, int kt, int slot) __attribute__((always_inline)) {
        const int kpos = k_reverse ? ksteps - 1 - kt : kt;
#pragma unroll
        for (int i = 0; i < kLoads; ++i)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(src[i], VDMQ_LDS_PTR(lds + slot * kStageBytes + (i * kWaves + wave) * 1024), 16,
                                                     lane_off[i], kpos * (KS / 64) * kBf6PanelKb, 0, 0);
    };
    struct Side {
        _Float16 as[2], ws, bias;
    };
    auto side_fetch = [&](int tile_m, int tile_n) __attribute__((always_inline)) {
        Side sd;
        const int m0 = tile_m * BM, n0 = tile_n * BN;
        const _Float16 *as_p = reinterpret_cast<const _Float16 *>(ascale);
        sd.as[0] = as_p[min(m0 + wm0 + lane, M - 1)];
        sd.as[1] = as_p[min(m0 + wm0 + 64 + lane, M - 1)];
        sd.ws = reinterpret_cast<const _Float16 *>(wscale)[min(n0 + wn0 + lane, N - 1)];
        sd.bias = static_cast<_Float16>(-0.0f);
        if (bias != nullptr) sd.bias = reinterpret_cast<const _Float16 *>(bias)[min(n0 + wn0 + lane, N - 1)];
        return sd;
    };
    uint8_t *side = lds + Cfg::kRingBytes + wave * kSideBytes;
    auto side_publish = [&](const Side &sd) __attribute__((always_inline)) {
        *reinterpret_cast<_Float16 *>(side + kSideAs + lane * 2) = sd.as[0];
        *reinterpret_cast<_Float16 *>(side + kSideAs + 128 + lane * 2) = sd.as[1];
        *reinterpret_cast<_Float16 *>(side + kSideWs + lane * 2) = sd.ws;
        *reinterpret_cast<_Float16 *>(side + kSideBias + lane * 2) = sd.bias;
    };
    const uint32_t la = lane * 16, lb = kBlkPlaneB + lane * 8;
    auto read = [&](v8i (&wf)[NI], v8i (&xf)[MI], const uint8_t *stage, int kb) __attribute__((always_inline)) {
#pragma unroll
        for (int ni = 0; ni < NI; ++ni) wf[ni] = ld_frag(stage + ((wn * NI + ni) * 2 + kb) * kBlkBytes, la, lb);
#pragma unroll
        for (int mi = 0; mi < MI; ++mi) xf[mi] = ld_frag(stage + ((BN / 32 + wm * MI + mi) * 2 + kb) * kBlkBytes, la, lb);
    };
    v16f acc[NI][MI];

    // (the first tile is found the long way: the table does not exist yet)
    int seq = -1, tile_m = -1, tile_n = 0, skipped = 0;
    do {
        if (!locate(++seq, tile_m, tile_n)) return; /* the same for the whole workgroup */
    } while (tile_m < 0);
    __amdgpu_buffer_rsrc_t src[kLoads];
    sources(src, tile_m, tile_n);
    bool k_reverse = tmap.contig && (seq & 1) != 0;
    {
        const Side sd = side_fetch(tile_m, tile_n);
#pragma unroll
        for (int s = 0; s < S; ++s)
            if (s < ksteps) issue(src, k_reverse, s, s);
        fill_tile_table();
        if (ksteps >= S) /* stages 0 and 1, as for every later tile; the table's writes */
            __builtin_amdgcn_s_waitcnt(waitcnt_imm(kLoads * (S - 2), 0));
        else
            __builtin_amdgcn_s_waitcnt(waitcnt_imm(0, 0));
        lds_barrier();
        side_publish(sd);
    }
    int cur = 0; /* ring slot of the tile's K step under work */
    v8i wfa[NI], xfa[MI], wfb[NI], xfb[MI];
    [[maybe_unused]] int dbg_tile = 0;
    for (;;) {
        const uint64_t tile_started = wall_clock64(); /* 100 MHz */
        VDMQ_STAMP(dbg_tile, 0);
        read(wfa, xfa, lds + cur * kStageBytes, 0);
        const Bf6KLoop<Cfg> k_loop{lds, src, lane_off, wave, wn, wm, la, lb, ksteps, k_reverse};
        k_loop.run(cur, acc, wfa, xfa, wfb, xfb);
        VDMQ_STAMP(dbg_tile, 1);

        // ---- the next tile: its first two K steps go into slots 1 and 2 now (every wave is past the last barrier of
        // the K loop, behind which nothing reads the ring any more); slot 0 holds the epilogue's staging.  Not so when
        // this place has no tile in the super-tile(s) that follow: a workgroup that went straight on would from then
        // on run a tile ahead of the rest of its XCD -- on another super-tile, whose operand slabs it would pull through
        // L2 alone (measured on N = 13824, 54 tile columns: half again as many bytes from beyond L2).  It sits those
        // super-tiles out, a tile's time each, and starts its next tile when the XCD's other workgroups do.
        const int m0 = tile_m * BM, n0 = tile_n * BN;
        int next_m = -1, next_n = 0;
        const bool more = next_tile(seq, next_m, next_n, skipped);
        const bool prefetch = more && skipped == 0;
        Side next_side = {};
        bool next_reverse = false;
        auto request_next = [&]() __attribute__((always_inline)) {
            sources(src, next_m, next_n);
            next_reverse = tmap.contig && (seq & 1) != 0;
            next_side = side_fetch(next_m, next_n);
            issue(src, next_reverse, 0, 1);
            if (ksteps > 1) issue(src, next_reverse, 1, 2);
        };
        if (prefetch) request_next();
        VDMQ_STAMP(dbg_tile, 2);

        // ---- fp16 epilogue of this tile.  The prefetched steps have to be in LDS, for every wave, before the next tile
        // reads them.  Loads and stores share one counter, so the wave waits for its loads before its first store --
        // by then they have had the first strip's conversion to arrive -- and the barrier below publishes them.
        auto prefetch_landed = [&] {
            if (prefetch) __builtin_amdgcn_s_waitcnt(waitcnt_imm(0, 15));
        };
        if (n0 + wn0 < N && m0 + wm0 < M) /* the same for the whole wave */
            bf6_epilogue<Cfg, STREAM_OUT, TAIL, BF16>(acc, side, lds + wave * Cfg::kStagingBytes, lane, m0 + wm0, n0 + wn0, out, ldo, M, N,
                                                      tail, prefetch_landed);
        else
            prefetch_landed();
        VDMQ_STAMP(dbg_tile, 3);
        if (!more) break;
        if (!prefetch) {
            const uint64_t now = wall_clock64(), until = now + static_cast<uint64_t>(skipped) * (now - tile_started);
            while (wall_clock64() < until) __builtin_amdgcn_s_sleep(32);
            request_next();
            __builtin_amdgcn_s_waitcnt(waitcnt_imm(0, 15));
        }
        __builtin_amdgcn_s_waitcnt(waitcnt_imm(63, 0)); /* the staging reads of this wave are done */
        lds_barrier();
        VDMQ_STAMP(dbg_tile, 4);
        ++dbg_tile;
        side_publish(next_side);
        if (ksteps > 2) issue(src, next_reverse, 2, 0);
        tile_m = next_m;
        tile_n = next_n;
        k_reverse = next_reverse;
        cur = 1;
    }
#endif
}

// bf6 code of an int4 value given as a two's complement nibble: q / 16 as an E3M2 float, which is sign << 5 | |q|
// (1/16 ... 3/16 are the format's denormals, 4/16 ... 8/16 its first normals)
__device__ __forceinline__ uint32_t bf6_code(uint32_t nib) {
    const int q = static_cast<int>(nib << 28) >> 28;
    return q < 0 ? 32u | static_cast<uint32_t>(-q) : static_cast<uint32_t>(q);
}

// int4 rows -> bf6 blocks; one thread per (row-block, k-block, lane).  The source is either native (row-major, low
// nibble = even k, rows of src_row_bytes) or, for V1, a checkpoint's weight buffer in the v1 word order
// (vdmq_layout.hip): the four 32-bit words that hold row n, k = 64 * kb + 32 * h + 8 * t ... + 7 (t = 0..3) are words
// 2 * (r / 8) + h of the 16-byte groups ((n / 128 * KG + kb) * 8 + n / 16 % 8) * 32 + 4 * (r % 8) + t, r = n % 16.
template <bool V1>
__global__ __launch_bounds__(256) void nibbles_to_bf6_kernel(const uint8_t *__restrict__ src, int64_t rows, int64_t src_row_bytes,
                                                             int kblocks, int src_kblocks, uint8_t *__restrict__ dst, int64_t total) {
    const int64_t idx = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (idx >= total) return;
    const int l = static_cast<int>(idx & 63);
    const int64_t blk = idx >> 6;
    const int kb = static_cast<int>(blk % kblocks);
    const int64_t rb = blk / kblocks;
    const int64_t r = rb * 32 + (l & 31);
    const int h = l >> 5;
    uint32_t regs[6] = {0, 0, 0, 0, 0, 0};
    if (r < rows && kb < src_kblocks) {
        uint32_t w[4];
        if (V1) {
            const int r16 = static_cast<int>(r & 15);
            const int64_t group = (((r >> 7) * src_kblocks + kb) * 8 + ((r >> 4) & 7)) * 32 + 4 * (r16 & 7);
            const uint32_t *words = reinterpret_cast<const uint32_t *>(src);
#pragma unroll
            for (int t = 0; t < 4; ++t) w[t] = words[(group + t) * 4 + 2 * (r16 >> 3) + h];
        } else {
            const u32x4 v = *reinterpret_cast<const u32x4 *>(src + r * src_row_bytes + kb * 32 + h * 16); /* 32 nibbles */
            w[0] = v.x, w[1] = v.y, w[2] = v.z, w[3] = v.w;
        }
#pragma unroll
        for (int e = 0; e < 32; ++e) {
            const uint64_t code = bf6_code((w[e / 8] >> (4 * (e % 8))) & 0xFu);
            const int bit = 6 * e, word = bit / 32, sh = bit % 32;
            regs[word] |= static_cast<uint32_t>(code << sh);
            if (sh > 26) regs[word + 1] |= static_cast<uint32_t>(code >> (32 - sh));
        }
    }
    *reinterpret_cast<u32x4 *>(dst + bf6_piece(rb * 32 + (l & 31), kb, h, false, kblocks)) = u32x4{regs[0], regs[1], regs[2], regs[3]};
    *reinterpret_cast<u32x2 *>(dst + bf6_piece(rb * 32 + (l & 31), kb, h, true, kblocks)) = u32x2{regs[4], regs[5]};
}

// bf6 weight blocks -> the checkpoint's v1 buffer: nibbles_to_bf6_kernel<true> backwards, one thread per (row-block,
// k-block, lane).  A thread decodes its 32 codes into four 32-bit words of eight nibbles and stores them where that
// kernel read them, so every word of the v1 buffer is written exactly once.
__global__ __launch_bounds__(256) void bf6_to_v1_kernel(const uint8_t *__restrict__ blocks, int64_t rows, int kblocks, int dst_kblocks,
                                                        uint8_t *__restrict__ dst, int64_t total) {
    const int64_t idx = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (idx >= total) return;
    const int l = static_cast<int>(idx & 63);
    const int64_t blk = idx >> 6;
    const int kb = static_cast<int>(blk % kblocks);
    const int64_t r = (blk / kblocks) * 32 + (l & 31);
    const int h = l >> 5;
    if (r >= rows || kb >= dst_kblocks) return; /* padding */
    const u32x4 a = *reinterpret_cast<const u32x4 *>(blocks + bf6_piece(r, kb, h, false, kblocks));
    const u32x2 b = *reinterpret_cast<const u32x2 *>(blocks + bf6_piece(r, kb, h, true, kblocks));
    const uint32_t regs[7] = {a.x, a.y, a.z, a.w, b.x, b.y, 0};
    uint32_t w[4] = {0, 0, 0, 0};
#pragma unroll
    for (int e = 0; e < 32; ++e) {
        const int bit = 6 * e, word = bit / 32, sh = bit % 32;
        uint32_t code = regs[word] >> sh;
        if (sh > 26) code |= regs[word + 1] << (32 - sh);
        const uint32_t mag = code & 31u; /* |q|, 0...8 */
        const uint32_t nib = (code & 32u) != 0 ? (0u - mag) & 0xFu : mag & 0xFu;
        w[e / 8] |= nib << (4 * (e % 8));
    }
    const int r16 = static_cast<int>(r & 15);
    const int64_t group = (((r >> 7) * dst_kblocks + kb) * 8 + ((r >> 4) & 7)) * 32 + 4 * (r16 & 7);
    uint32_t *words = reinterpret_cast<uint32_t *>(dst);
#pragma unroll
    for (int t = 0; t < 4; ++t) words[(group + t) * 4 + 2 * (r16 >> 3) + h] = w[t];
}

}  // namespace

#ifdef VDMQ_DBG_TIMELINE
extern "C" int vdmq_debug_timeline(void *host_out, int clear) {
    if (clear) {
        void *p = nullptr;
        if (hipGetSymbolAddress(&p, HIP_SYMBOL(g_timeline)) != hipSuccess) return -1;
        return hipMemset(p, 0, sizeof(uint64_t) * 256 * 64 * 6) == hipSuccess ? 0 : -1;
    }
    return hipMemcpyFromSymbol(host_out, HIP_SYMBOL(g_timeline), sizeof(uint64_t) * 256 * 64 * 6) == hipSuccess ? 0 : -1;
}
#endif

int64_t bf6_kblocks(int64_t K) { return (K + 127) / 128 * 2; }
int64_t bf6_bytes(int64_t rows, int64_t K) { return (rows + 31) / 32 * bf6_kblocks(K) * kBlkBytes; }

int launch_nibbles_to_bf6(const uint8_t *native, int64_t rows, int64_t K, uint8_t *blocks, hipStream_t s) {
    if (rows == 0) return VDMQ_OK;
    const int64_t kblocks = bf6_kblocks(K);
    const int64_t total = (rows + 31) / 32 * kblocks * 64;
    hipLaunchKernelGGL(nibbles_to_bf6_kernel<false>, dim3(static_cast<unsigned>(ceil_div(total, 256))), dim3(256), 0, s, native, rows,
                       k_padded(K) / 2, static_cast<int>(kblocks), static_cast<int>(k_padded(K) / 64), blocks, total);
    return check_launch("nibbles_to_bf6_kernel");
}

int launch_weight_v1_to_bf6(const uint8_t *qweight_v1, int64_t N, int64_t K, uint8_t *blocks, hipStream_t s) {
    if (N == 0) return VDMQ_OK;
    const int64_t kblocks = bf6_kblocks(K);
    const int64_t total = (N + 31) / 32 * kblocks * 64;
    hipLaunchKernelGGL(nibbles_to_bf6_kernel<true>, dim3(static_cast<unsigned>(ceil_div(total, 256))), dim3(256), 0, s, qweight_v1, N,
                       K / 2, static_cast<int>(kblocks), static_cast<int>(K / 64), blocks, total);
    return check_launch("nibbles_to_bf6_kernel");
}

int launch_bf6_to_weight_v1(const uint8_t *blocks, int64_t N, int64_t K, uint8_t *qweight_v1, hipStream_t s) {
    if (N == 0) return VDMQ_OK;
    const int64_t kblocks = bf6_kblocks(K);
    const int64_t total = (N + 31) / 32 * kblocks * 64;
    hipLaunchKernelGGL(bf6_to_v1_kernel, dim3(static_cast<unsigned>(ceil_div(total, 256))), dim3(256), 0, s, blocks, N, static_cast<int>(kblocks),
                       static_cast<int>(K / 64), qweight_v1, total);
    return check_launch("bf6_to_v1_kernel");
}

namespace {

template <class Cfg>
int launch_bf6_cfg(const uint8_t *xblocks, const __half *ascale, const uint8_t *wblocks, const __half *wscale, const __half *bias,
                   __half *out, bool out_bf16, int32_t *acc_out, int64_t M, int64_t N, int64_t K, int64_t ldo, const GemmTail &tail,
                   hipStream_t s) {
    const int tiles_m = static_cast<int>(ceil_div(M, Cfg::BM)), tiles_n = static_cast<int>(ceil_div(N, Cfg::BN));
    // Places per super-tile: what an XCD's CUs hold at once.  The small configuration's problems are few such
    // super-tiles, mostly partly empty ones (M = 512: 4 tile rows in a shape of 16 x 4, so 16 tiles per super-tile);
    // measured against both alternatives on M = 512, K = 5120, N = 10240 (320 tiles; 25.8 us as it is): the edges
    // regrouped into five full super-tiles 28.1 us, super-tiles of four dealt over all XCDs 31.7 us (K = 3072, N = 6144:
    // 11.2 / 18.2 / 13.2 us) -- two workgroups that share a CU keep its matrix pipes busier than one each on two CUs,
    // and five XCDs are too few.
    constexpr int per_log2 = Cfg::kPerLog2, per = 1 << per_log2;
    // Super-tile shape.  Candidates in order of preference: 8 x 4 tiles (2048 token rows x 1024 weight rows, the
    // fewest operand bytes per tile and measured best wherever the work is even), the same with the edge super-tiles
    // regrouped (fuller, so fewer of them), 16 x 2, 16 x 2 regrouped.  A later one replaces an earlier one when it
    // saves the XCDs a round (super-tiles go round the XCDs in turn, and a workgroup that walks tiles spends a round
    // on each, however full: six tile columns at M = 32760 take 4 rounds as 8 x 4 and 8 x 2, 3 with the last two
    // columns as 16 x 2; M = 75600, N = 13824, 54 tile columns: 37 half-empty super-tiles become 19 full ones,
    // 65 -> 63 rounds; M = 27280, N = 14336, three tile rows left over: 25 -> 24) or, at the same number of rounds,
    // takes a tenth off the busiest XCD's tile count.  Problems of less than two tiles per CU keep their partly empty
    // edge super-tiles: the few tiles are better spread over all XCDs than packed into the places of some.
    const bool small = static_cast<int64_t>(tiles_m) * tiles_n < 2 * kXcds * per;
    Bf6TileMap tm;
    int64_t best_load = -1, best_rounds = 0;
    for (int variant = 0; variant < 4; variant += small ? 2 : 1) {
        Bf6TileMap cand;
        bf6_tilemap_shape(cand, tiles_m, tiles_n, per_log2, 2 - variant / 2, variant % 2 != 0);
        int64_t load[kXcds] = {};
        const bool modelled = cand.total_super <= 4096; /* beyond that the edges no longer matter: the first shape is taken */
        if (modelled)
            for (int st = 0; st < cand.total_super; ++st)
                load[st % kXcds] += bf6_tilemap_tiles_before(cand, st + 1) - bf6_tilemap_tiles_before(cand, st);
        int64_t worst = 0;
        for (int x = 0; x < kXcds; ++x) worst = load[x] > worst ? load[x] : worst;
        const int64_t cand_rounds = ceil_div(cand.total_super, kXcds);
        if (best_load < 0 || (modelled && best_load > 0 &&
                              ((!small && cand_rounds < best_rounds) || ((small || cand_rounds == best_rounds) && worst * 10 <= best_load * 9)))) {
            best_load = worst;
            best_rounds = cand_rounds;
            tm = cand;
        }
    }
    const int64_t total_super = tm.total_super;
    if (best_load < 0 || total_super * per + kXcds * per > (int64_t(1) << 30))
        return fail(VDMQ_ESHAPE, "M x N = %lld x %lld needs more workgroups than one launch can hold", (long long)M, (long long)N);
    tm.contig = 0;
    for (int x = 0; x <= kXcds; ++x) tm.start[x] = 0;
    int rounds = static_cast<int>(ceil_div(total_super, kXcds));
    // Long K and wide N: every XCD takes one contiguous run of the super-tile sequence (n fastest); consecutive
    // super-tiles of an XCD then share their token rows and, walking K in opposite directions, re-use what the
    // previous one left in L2 (as in vdmq_gemm.hip).  Measured at M = 75600, K = 5120: 12...14 % fewer bytes from
    // beyond L2 and 0...2 % less time for N = 13824 and 15360; with 20 tile columns or fewer (N = 5120, 3072) it
    // fetches 4 % more and is 3...5 % slower than taking turns.
    const bool contig = K >= 2048 && tm.tiles_n >= 48;
    if (contig) rounds = bf6_tilemap_runs(tm, true);
    const dim3 grid(static_cast<unsigned>(rounds) * kXcds * per), block(Cfg::kWaves * 64);
    const bool stream_out = M * N * 2 > (int64_t(224) << 20);
    const bool has_tail = tail.gate != nullptr || tail.residual != nullptr;
    const int which = acc_out != nullptr ? 2 : (stream_out ? 1 : 0) + (has_tail ? 3 : out_bf16 ? 5 : 0); /* (a tail comes with fp16 only) */
    using Kernel = void (*)(const uint8_t *, const uint8_t *, const __half *, const __half *, const __half *, __half *, int32_t *, int, int,
                            int, int64_t, Bf6TileMap, GemmTail);
    const Kernel kernels[7] = {gemm_bf6_kernel<Cfg, 0>, gemm_bf6_kernel<Cfg, 1>, gemm_bf6_kernel<Cfg, 2>, gemm_bf6_kernel<Cfg, 3>,
                               gemm_bf6_kernel<Cfg, 4>, gemm_bf6_kernel<Cfg, 5>, gemm_bf6_kernel<Cfg, 6>};
    constexpr int kMaxDevices = 64;
    static bool attr_done[kMaxDevices][7] = {};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return fail(VDMQ_ELAUNCH, "no current HIP device");
    if (!attr_done[dev][which]) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kernels[which]), hipFuncAttributeMaxDynamicSharedMemorySize,
                                           Cfg::kLdsBytesOneTile);
        if (e != hipSuccess) return fail(VDMQ_ELAUNCH, "hipFuncSetAttribute(%d bytes of LDS): %s", Cfg::kLdsBytesOneTile, hipGetErrorString(e));
        attr_done[dev][which] = true;
    }
    // The persistent kernel gives every CU position a fixed share -- its place in each super-tile of the XCD's
    // sequence -- where the hardware dispatcher would refill a CU as soon as it is free: it pays when few super-tiles
    // are partly empty (each costs its XCD a whole round: before the edges were regrouped, M = 27280, N = 14336 took a
    // third more rounds with the ragged last row in one XCD's run and ran 16 % slower), i.e. when its rounds are
    // within 15 % of the busiest XCD's tiles / places (M = 32760, N = 4608: 10 rounds for 9, still +4 %).  Every fp16
    // output mode has it (with the gated residual tail: 249 registers, +3...4 % on the 14B and 5B output projections).
    const int64_t all_tiles = static_cast<int64_t>(tm.tiles_m) * tm.tiles_n;
    const int64_t busiest = tm.contig || best_load == 0 ? ceil_div(all_tiles, kXcds) : best_load;
    // (one workgroup per CU position: only where the device has as many CUs as the kernel has positions; elsewhere the
    // hardware dispatcher places the one-tile workgroups)
    static int cu_count[kMaxDevices] = {};
    if (cu_count[dev] == 0 && hipDeviceGetAttribute(&cu_count[dev], hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) cu_count[dev] = -1;
    // (its contiguous runs hold equal numbers of super-tiles: a round each, however full)
    const int64_t rounds_p = ceil_div(total_super, kXcds);
    const bool persistent = Cfg::kOcc == 1 && which != 2 && cu_count[dev] == kXcds * per && rounds_p * 100 <= ceil_div(busiest, per) * 115;
    if constexpr (Cfg::kOcc == 1) if (persistent) {
        if (contig) bf6_tilemap_runs(tm, false);
        using PKernel = void (*)(const uint8_t *, const uint8_t *, const __half *, const __half *, const __half *, __half *, int, int, int,
                                 int64_t, Bf6TileMap, GemmTail);
        const PKernel pk[7] = {gemm_bf6_persistent_kernel<Cfg, 0>, gemm_bf6_persistent_kernel<Cfg, 1>, nullptr, gemm_bf6_persistent_kernel<Cfg, 3>,
                               gemm_bf6_persistent_kernel<Cfg, 4>, gemm_bf6_persistent_kernel<Cfg, 5>, gemm_bf6_persistent_kernel<Cfg, 6>};
        static bool pattr[kMaxDevices][7] = {};
        if (!pattr[dev][which]) {
            hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(pk[which]), hipFuncAttributeMaxDynamicSharedMemorySize,
                                               Cfg::kLdsBytes);
            if (e != hipSuccess) return fail(VDMQ_ELAUNCH, "hipFuncSetAttribute: %s", hipGetErrorString(e));
            pattr[dev][which] = true;
        }
        hipLaunchKernelGGL(pk[which], dim3(kXcds * per), block, Cfg::kLdsBytes, s, xblocks, wblocks, ascale, wscale, bias, out,
                           static_cast<int>(M), static_cast<int>(N), static_cast<int>(bf6_kblocks(K)), ldo, tm, tail);
        const int rc = check_launch("gemm_bf6_persistent_kernel");
        if (rc == VDMQ_OK)
            record_gemm_launch({VDMQ_KERNEL_GEMM_BF6_PERSISTENT, Cfg::BM, Cfg::BN, per >> tm.group_n_log2, 1 << tm.group_n_log2, tm.contig,
                                static_cast<int64_t>(kXcds * per)});
        return rc;
    }
    hipLaunchKernelGGL(kernels[which], grid, block, Cfg::kLdsBytesOneTile, s, xblocks, wblocks, ascale, wscale, bias, out, acc_out,
                       static_cast<int>(M), static_cast<int>(N), static_cast<int>(bf6_kblocks(K)), ldo, tm, tail);
    const int rc = check_launch("gemm_bf6_kernel");
    if (rc == VDMQ_OK)
        record_gemm_launch({VDMQ_KERNEL_GEMM_BF6, Cfg::BM, Cfg::BN, per >> tm.group_n_log2, 1 << tm.group_n_log2, tm.contig,
                            static_cast<int64_t>(grid.x)});
    return rc;
}

}  // namespace

int launch_gemm_bf6(const uint8_t *xblocks, const __half *ascale, const uint8_t *wblocks, const __half *wscale, const __half *bias,
                    void *out, int out_dtype, int32_t *acc_out, int64_t M, int64_t N, int64_t K, int64_t ldo, const GemmTail &tail,
                    hipStream_t s) {
    if (M == 0 || N == 0) return VDMQ_OK;
    // (both 16-bit output types go through the same staging and stores; the kernels take the pointer as fp16)
    // Problems of at most half a 256 x 256 tile per CU take 128 x 128 tiles, two workgroups of four waves per CU: four
    // times as many workgroups for the same K loop.  Measured on 150 shapes (M 1...32768, N 128...15360, K 64...13824):
    // up to 128 big tiles the small ones take 0.46...0.9 of the time (512 x 5120 -> 10240: 28 -> 25 us, 512 x 1536 ->
    // 3072: 13.7 -> 7.3 us), from 160 on 1.0...1.4.
    if (ceil_div(M, Bf6Big::BM) * ceil_div(N, Bf6Big::BN) <= kXcds * 32 / 2)
        return launch_bf6_cfg<Bf6Small>(xblocks, ascale, wblocks, wscale, bias, static_cast<__half *>(out), out_dtype == VDMQ_OUT_BF16, acc_out, M,
                                        N, K, ldo, tail, s);
    return launch_bf6_cfg<Bf6Big>(xblocks, ascale, wblocks, wscale, bias, static_cast<__half *>(out), out_dtype == VDMQ_OUT_BF16, acc_out, M, N,
                                  K, ldo, tail, s);
}

}  // namespace vdmq
