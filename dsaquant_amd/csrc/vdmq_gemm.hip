// W4A4 GEMM for gfx950 (CDNA4 has no int4 MFMA).
//
//   acc[m,n] = sum_k qx[m,k] * qw[n,k]   exact int32
//   out[m,n] = fp16(float(acc) * (float(as[m]) * float(ws[n]))) (+ bias[n] in fp16)
//
// Data path.  Both operands are row-major packed int4; a K step takes 128 or
// 256 k (64 or 128 bytes) of every row.  A workgroup owns a BM x BN output tile and walks K through
// a ring of LDS stages filled by 128-bit direct-to-LDS loads
// (buffer_load_dwordx4 ... lds: no VGPR staging, no ds_write).  A lane reads 16
// bytes (32 nibbles) of one row from LDS and widens each 32-bit word p into two
// MFMA operand registers
//     lo = (p << 4) & 0xF0F0F0F0   (even-k nibbles, as int8 = 16*q)
//     hi =  p       & 0xF0F0F0F0   (odd-k nibbles,  as int8 = 16*q)
// Both operands are widened the same way, so k pairs up correctly whatever
// order the MFMA consumes the bytes in, and v_mfma_i32_32x32x32_i8 accumulates
// 256 * sum(qx*qw) exactly (|16q| <= 128, K <= 65536 keeps |acc| < 2^31).
// The epilogue folds the factor 1/256 (a power of two, exact) into the scale.
//
// MFMA orientation: the A operand holds weight rows (n), the B operand token
// rows (m), so a lane's four consecutive accumulator registers are four
// consecutive n of one token: an 8-byte fp16 store.
//
// LDS layout of a stage: rows 0..BN-1 are weight rows, BN..BN+BM-1 token rows,
// 64 or 128 bytes each; the 16-byte pieces of row r are stored at piece index
// p ^ ((r/4)%4) (four pieces) or p ^ ((r/2)%8) (eight), which makes the 16
// lanes of a ds_read_b128 phase hit 16 different bank groups (measured: zero
// bank conflicts).
//
// Synchronisation: the direct-to-LDS loads are tracked by vmcnt only and the
// stage ring is published with raw s_barrier (no fence: a workgroup fence
// would drain every load in flight), so the waits are written by hand below.
#include <type_traits>

#include "vdmq_internal.h"

namespace vdmq {
namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));

#define VDMQ_GLOBAL_PTR(p) ((const __attribute__((address_space(1))) void *)(p))
#define VDMQ_LDS_PTR(p) ((__attribute__((address_space(3))) void *)(p))


// s_waitcnt immediate for gfx9: vmcnt[3:0] | expcnt[6:4] | lgkmcnt[11:8] | vmcnt[15:14]
[[maybe_unused]] constexpr int waitcnt_imm(int vm, int lgkm) { return (vm & 15) | ((vm >> 4) << 14) | (7 << 4) | ((lgkm & 15) << 8); }

[[maybe_unused]] __device__ __forceinline__ void lds_barrier() {
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
}

[[maybe_unused]] __device__ __forceinline__ v4i widen(uint32_t p0, uint32_t p1) {
    v4i r;
    r[0] = static_cast<int>((p0 << 4) & 0xF0F0F0F0u);
    r[1] = static_cast<int>(p0 & 0xF0F0F0F0u);
    r[2] = static_cast<int>((p1 << 4) & 0xF0F0F0F0u);
    r[3] = static_cast<int>(p1 & 0xF0F0F0F0u);
    return r;
}

template <int BM_, int BN_, int WAVES_M_, int WAVES_N_, int STAGES_, int OCC_ = 1, int KSTEP_ = 128>
struct GemmCfg {
    static constexpr int kOccupancy = OCC_; /* workgroups per CU the register budget must allow */
    static constexpr int kKStepElems = KSTEP_;       /* k per LDS stage: 128 or 256 */
    static constexpr int kRowBytes = KSTEP_ / 2;     /* bytes of one operand row per stage */
    static constexpr int kPieces = kRowBytes / 16;   /* 16-byte pieces per row: 4 or 8 */
    static constexpr int kReads = kPieces / 2;       /* 128-bit fragment reads per lane and stage */
    static constexpr int kSwzShift = kPieces == 4 ? 2 : 1; /* piece index is XORed with (row >> shift) % kPieces */
    static constexpr int kDmaRows = 64 / kPieces;    /* rows filled by one direct-to-LDS wave instruction */
    static_assert(KSTEP_ == 128 || KSTEP_ == 256, "K step");
    static_assert(kKStep % KSTEP_ == 0, "native rows are padded to kKStep");
    static constexpr int BM = BM_, BN = BN_, WAVES_M = WAVES_M_, WAVES_N = WAVES_N_, STAGES = STAGES_;
    static constexpr int kWaves = WAVES_M * WAVES_N;
    static constexpr int kThreads = kWaves * kWaveSize;
    static constexpr int kWaveM = BM / WAVES_M;
    static constexpr int kWaveN = BN / WAVES_N;
    static constexpr int kMI = kWaveM / 32;
    static constexpr int kNI = kWaveN / 32;
    static constexpr int kRows = BM + BN;
    static constexpr int kStageBytes = kRows * kRowBytes;
    static constexpr int kRingBytes = kStageBytes * STAGES;
    // beside the ring, per wave: the fp16 token scales of its rows, the channel scales and the bias of its columns,
    // fetched when the tile starts so that the fp16 epilogue does not wait for them
    static constexpr int kSideAs = 0, kSideWs = 2 * kWaveM, kSideBias = 2 * kWaveM + 2 * kWaveN, kSideBytes = 2 * kWaveM + 4 * kWaveN;
    static constexpr int kLdsBytes = kRingBytes + kWaves * kSideBytes;
    // one direct-to-LDS instruction of one wave fills kDmaRows rows (1 KiB)
    static constexpr int kRowBlocks = kRows / kDmaRows;
    static constexpr int kLoads = kRowBlocks / kWaves; /* per wave (= per lane) and stage */
    // epilogue staging: one 32-row strip of the wave tile as fp16, rows padded by 16 bytes
    static constexpr int kStageRowBytes = kWaveN * 2 + 16;
    static constexpr int kStagingBytes = 32 * kStageRowBytes;
    static constexpr int kPiecesPerRow = kWaveN / 8; /* 16-byte pieces of one strip row */
    static_assert(kStagingBytes * kWaves <= kStageBytes * STAGES_, "epilogue staging reuses the stage ring");
    static_assert(kWaveN <= 64, "one lane per column fetches the channel scale and the bias");
    static_assert(kWaveN == 64, "an output split by blocks of 64 columns keeps a wave's stores inside one part");
    static_assert(kRowBlocks % kWaves == 0, "row blocks must divide evenly over the waves");
    static_assert(BN % kDmaRows == 0 && kWaveM % 32 == 0 && kWaveN % 32 == 0, "tile shape");
    static_assert(kLoads * (STAGES - 1) < 64, "vmcnt is a 6-bit counter");
};

// Issue the direct-to-LDS loads of one stage.  `woff`/`xoff` are per-lane byte
// offsets (clamped to valid rows) from the wave-uniform bases.
#if defined(__HIP_DEVICE_COMPILE__) /* (the host pass does not know the buffer builtins) */
// A buffer load takes its address in three parts -- the tile's first row (shared resource), the K position (scalar
// offset) and the lane's row and piece (vector offset, fixed for the whole tile) -- so the K loop spends no vector
// instruction on addresses; global_load_lds wants a 64-bit address per lane.
template <typename Cfg>
__device__ __forceinline__ void issue_stage(__amdgpu_buffer_rsrc_t wsrc, __amdgpu_buffer_rsrc_t xsrc, int koff,
                                            const uint32_t (&off)[Cfg::kLoads], uint8_t *lds_stage, int wave) {
#pragma unroll
    for (int i = 0; i < Cfg::kLoads; ++i) {
        const int rb = i * Cfg::kWaves + wave; /* wave-uniform row block */
        __builtin_amdgcn_raw_ptr_buffer_load_lds((rb * Cfg::kDmaRows < Cfg::BN) ? wsrc : xsrc, VDMQ_LDS_PTR(lds_stage + rb * 1024), 16, off[i],
                                                 koff, 0, 0);
    }
}
#endif

template <typename Cfg>
__device__ __forceinline__ void read_frags(u32x4 (&wf)[Cfg::kNI], u32x4 (&xf)[Cfg::kMI], const uint8_t *lds_stage, uint32_t waddr,
                                           uint32_t xaddr) {
#pragma unroll
    for (int ni = 0; ni < Cfg::kNI; ++ni) wf[ni] = *reinterpret_cast<const u32x4 *>(lds_stage + waddr + ni * 32 * Cfg::kRowBytes);
#pragma unroll
    for (int mi = 0; mi < Cfg::kMI; ++mi) xf[mi] = *reinterpret_cast<const u32x4 *>(lds_stage + xaddr + mi * 32 * Cfg::kRowBytes);
}

// Operand registers of one K=32 MFMA step for the whole wave tile.
template <typename Cfg>
struct Operands {
    v4i a[Cfg::kNI]; /* weight rows */
    v4i b[Cfg::kMI]; /* token rows */
};

template <typename Cfg, int HALF>
__device__ __forceinline__ void widen_frags(Operands<Cfg> &o, const u32x4 (&wf)[Cfg::kNI], const u32x4 (&xf)[Cfg::kMI]) {
#pragma unroll
    for (int ni = 0; ni < Cfg::kNI; ++ni) o.a[ni] = HALF ? widen(wf[ni].z, wf[ni].w) : widen(wf[ni].x, wf[ni].y);
#pragma unroll
    for (int mi = 0; mi < Cfg::kMI; ++mi) o.b[mi] = HALF ? widen(xf[mi].z, xf[mi].w) : widen(xf[mi].x, xf[mi].y);
}

template <typename Cfg>
__device__ __forceinline__ void mma_step(v16i (&acc)[Cfg::kNI][Cfg::kMI], const Operands<Cfg> &o) {
#pragma unroll
    for (int ni = 0; ni < Cfg::kNI; ++ni)
#pragma unroll
        for (int mi = 0; mi < Cfg::kMI; ++mi) acc[ni][mi] = __builtin_amdgcn_mfma_i32_32x32x32_i8(o.a[ni], o.b[mi], acc[ni][mi], 0, 0, 0);
}

// Instruction-mix hints.  A read's work is split into two scheduling regions of
// kNI*kMI MFMAs each (closed by a full scheduling barrier, so the scheduler
// cannot pile one region's widening ops up in the other): every MFMA is
// followed by its share of the widening VALU ops (4.5 per MFMA for a 128 x 64
// wave tile: 4 and 5 alternately); the LDS reads ride on the first MFMAs of the first region, the
// direct-to-LDS loads on those of the second.
template <typename Cfg, int NDS, int NVMEM, int I = 0>
__device__ __forceinline__ void schedule_region() {
    constexpr int kMfma = Cfg::kNI * Cfg::kMI;
    constexpr int kValu = (Cfg::kNI + Cfg::kMI) * 6; /* widening ops of the region */
    if constexpr (I < kMfma) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0); /* MFMA */
        if constexpr (I < NDS) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0); /* DS read */
        if constexpr (I < NVMEM) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0); /* VMEM read */
        __builtin_amdgcn_sched_group_barrier(0x002, kValu * (I + 1) / kMfma - kValu * I / kMfma, 0); /* VALU */
        schedule_region<Cfg, NDS, NVMEM, I + 1>();
    } else {
        __builtin_amdgcn_sched_barrier(0);
    }
}

// Tile order.  Workgroups are dealt round-robin to the 8 XCDs (each with its own
// L2), so workgroup b runs on XCD b%8 as its (b/8)-th.  Each XCD walks
// "super-tiles" of kGroupM x kGroupN tiles (32 = its CU count): the tiles that are
// resident on an XCD together share kGroupM token row-blocks and kGroupN weight
// row-blocks.
constexpr int kXcds = 8, kGroupM = 8, kGroupN = 4;

struct TileMap {
    int tiles_m, tiles_n, super_n;
    int start[kXcds + 1]; /* XCD x walks super-tiles [start[x], start[x+1]) */
    int contig;           /* 1: those contiguous runs; 0: super-tiles dealt round-robin (start[kXcds] = their number) */
};

[[maybe_unused]] __device__ __forceinline__ bool map_tile(const TileMap &tm, int bid, int &tile_m, int &tile_n) {
    const int xcd = bid % kXcds, slot = bid / kXcds;
    const int per = kGroupM * kGroupN;
    const int j = slot % per;
    int st;
    if (tm.contig) {
        // An XCD walks a contiguous run of super-tiles, n fastest: consecutive ones share their token
        // slab, and with the K walk reversed on every other one (see the kernel) the part of that slab
        // read last is still in this XCD's L2 when the next super-tile starts there.  The runs hold
        // equal numbers of tiles, not of super-tiles (those on the ragged edges are partly empty).
        st = tm.start[xcd] + slot / per;
        if (st >= tm.start[xcd + 1]) return false;
    } else {
        // super-tiles dealt round-robin: the 8 XCDs work on neighbouring super-tiles at any moment
        st = (slot / per) * kXcds + xcd;
        if (st >= tm.start[kXcds]) return false;
    }
    tile_m = (st / tm.super_n) * kGroupM + j / kGroupN;
    tile_n = (st % tm.super_n) * kGroupN + j % kGroupN;
    return tile_m < tm.tiles_m && tile_n < tm.tiles_n;
}

// OUT_MODE: 0 = scaled output, 1 = scaled output with non-temporal stores, 2 = raw int32 accumulators,
// 3 / 4 = 0 / 1 followed by the gated residual update (a separate instantiation: carrying the tail's
// branches and registers costs the plain kernel 1 %)
template <typename Cfg, int OUT_MODE>
__global__ __launch_bounds__(Cfg::kThreads, Cfg::kOccupancy * Cfg::kWaves / 4) void gemm_w4a4_kernel(const uint8_t *__restrict__ A, const uint8_t *__restrict__ W,
                                                                  const __half *__restrict__ ascale, const __half *__restrict__ wscale,
                                                                  const __half *__restrict__ bias, void *out, int out_dtype,
                                                                  int32_t *__restrict__ acc_out, int M, int N, int ldk, int64_t ldo,
                                                                  TileMap tmap, GemmTail tail) {
#if defined(__HIP_DEVICE_COMPILE__) /* the host pass needs the kernel's stub only */
    constexpr int BM = Cfg::BM, BN = Cfg::BN, S = Cfg::STAGES, L = Cfg::kLoads;
    constexpr bool ACC_OUT = OUT_MODE == 2, STREAM_OUT = OUT_MODE == 1 || OUT_MODE == 4, TAIL = OUT_MODE >= 3;
    extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];

    int tile_m, tile_n;
    if (!map_tile(tmap, blockIdx.x, tile_m, tile_n)) return;
    const int m0 = tile_m * BM, n0 = tile_n * BN;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int wm0 = (wave / Cfg::WAVES_N) * Cfg::kWaveM; /* within the tile */
    const int wn0 = (wave % Cfg::WAVES_N) * Cfg::kWaveN;
    const int l32 = lane & 31, lh = lane >> 5;

    constexpr int RB = Cfg::kRowBytes, R = Cfg::kReads;
    // ---- global -> LDS: per-lane source offsets (rows clamped into range: rows
    // beyond M or N are loaded from the last valid row and never stored)
    uint32_t goff[L];
    {
        const int wrows = min(BN, N - n0), xrows = min(BM, M - m0);
#pragma unroll
        for (int i = 0; i < L; ++i) {
            const int r = (i * Cfg::kWaves + wave) * Cfg::kDmaRows + lane / Cfg::kPieces; /* stage row this lane fills */
            const int piece = (lane % Cfg::kPieces) ^ ((r >> Cfg::kSwzShift) % Cfg::kPieces);
            const int rr = r < BN ? min(r, wrows - 1) : min(r - BN, xrows - 1);
            goff[i] = static_cast<uint32_t>(rr) * static_cast<uint32_t>(ldk) + piece * 16;
        }
    }
    // (rows of the tile that exist) x (bytes per row) each: the offsets above stay inside
    const __amdgpu_buffer_rsrc_t wsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t *>(W + static_cast<int64_t>(n0) * ldk), 0,
                                                                          min(BN, N - n0) * ldk, 0x00020000 /* raw buffer of dwords */);
    const __amdgpu_buffer_rsrc_t xsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t *>(A + static_cast<int64_t>(m0) * ldk), 0,
                                                                          min(BM, M - m0) * ldk, 0x00020000);

    // ---- LDS -> registers: per-lane fragment addresses for the R 128-bit reads
    // (j) of a stage; lanes 32..63 take the odd pieces.  Tile row offsets are
    // multiples of 32, so the swizzle term only depends on the lane.
    const int swz = (l32 >> Cfg::kSwzShift) % Cfg::kPieces;
    uint32_t waddr[R], xaddr[R];
#pragma unroll
    for (int j = 0; j < R; ++j) {
        const int piece = ((2 * j + lh) ^ swz) << 4;
        waddr[j] = (wn0 + l32) * RB + piece;
        xaddr[j] = (BN + wm0 + l32) * RB + piece;
    }

    v16i acc[Cfg::kNI][Cfg::kMI];
#pragma unroll
    for (int ni = 0; ni < Cfg::kNI; ++ni)
#pragma unroll
        for (int mi = 0; mi < Cfg::kMI; ++mi)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[ni][mi][r] = 0;

    const int ksteps = ldk / RB;
    // Every other workgroup of a CU slot walks K backwards: the end of the previous tile's operand
    // slabs is still in L2 when the next tile, which shares the token slab, starts there (measured:
    // 18 % fewer bytes fetched from beyond L2, 23 % for the widest shape).  Integer accumulation is
    // exact in any order.
    const bool k_reverse = tmap.contig && ((blockIdx.x / (kXcds * kGroupM * kGroupN)) & 1) != 0;
    auto kpos = [&](int kt) { return k_reverse ? ksteps - 1 - kt : kt; };

    uint8_t *side = lds + Cfg::kRingBytes + wave * Cfg::kSideBytes;
    const bool f16_out = !ACC_OUT && out_dtype == VDMQ_OUT_F16;
    // (no bias: -0, the one fp16 value whose addition changes no bit of any output)
    _Float16 side_as[(Cfg::kWaveM + 63) / 64] = {}, side_ws = 0, side_bias = static_cast<_Float16>(-0.0f);
    if (f16_out) { /* older than the stage loads below: complete before the first of those is waited for */
#pragma unroll
        for (int i = 0; i < (Cfg::kWaveM + 63) / 64; ++i)
            side_as[i] = reinterpret_cast<const _Float16 *>(ascale)[min(m0 + wm0 + i * 64 + lane, M - 1)];
        side_ws = reinterpret_cast<const _Float16 *>(wscale)[min(n0 + wn0 + (lane & (Cfg::kWaveN - 1)), N - 1)];
        if (bias != nullptr) side_bias = reinterpret_cast<const _Float16 *>(bias)[min(n0 + wn0 + (lane & (Cfg::kWaveN - 1)), N - 1)];
    }
    // prologue: fill the ring (as far as K reaches), wait for stage 0
#pragma unroll
    for (int s = 0; s < S; ++s)
        if (s < ksteps) issue_stage<Cfg>(wsrc, xsrc, kpos(s) * RB, goff, lds + s * Cfg::kStageBytes, wave);
    if (ksteps >= S)
        __builtin_amdgcn_s_waitcnt(waitcnt_imm(L * (S - 1), 15));
    else
        __builtin_amdgcn_s_waitcnt(waitcnt_imm(0, 15));
    lds_barrier();
    if (f16_out) { /* wave-private: the epilogue's reads follow these writes in the wave's own LDS queue */
#pragma unroll
        for (int i = 0; i < (Cfg::kWaveM + 63) / 64; ++i)
            if (i * 64 + lane < Cfg::kWaveM) *reinterpret_cast<_Float16 *>(side + Cfg::kSideAs + (i * 64 + lane) * 2) = side_as[i];
        if (lane < Cfg::kWaveN) {
            *reinterpret_cast<_Float16 *>(side + Cfg::kSideWs + lane * 2) = side_ws;
            *reinterpret_cast<_Float16 *>(side + Cfg::kSideBias + lane * 2) = side_bias;
        }
    }

    // Software pipeline.  fa/fb hold the raw LDS fragments of the 128-bit read
    // being consumed and of the next one; `lo` holds the widened first half of
    // the fragment about to be consumed, prepared one step ahead.
    u32x4 wfa[Cfg::kNI], xfa[Cfg::kMI], wfb[Cfg::kNI], xfb[Cfg::kMI];
    Operands<Cfg> lo, hi;
    read_frags<Cfg>(wfa, xfa, lds, waddr[0], xaddr[0]);
    widen_frags<Cfg, 0>(lo, wfa, xfa);

    // One stage (K step).  STEADY: stage kt+S exists (so the slot is refilled,
    // S-1 stages are in flight at the wait, and a next stage exists) -- a
    // branch-free body the scheduler can interleave as one region per read.
    // Read j of the stage is consumed while read j+1 (or read 0 of the next
    // stage) is fetched; the ring is published by ONE barrier per stage, placed
    // before the last read's MFMAs: by then every wave has finished its LDS
    // reads of the stage, so its slot can be refilled.
    int cur = 0; /* ring slot of stage kt */
    auto k_step = [&](int kt, auto steady_tag) {
        constexpr bool STEADY = decltype(steady_tag)::value;
        const uint8_t *stage = lds + cur * Cfg::kStageBytes;
        const int nxt = cur + 1 == S ? 0 : cur + 1;
#pragma unroll
        for (int j = 0; j < R; ++j) {
            // fragments alternate between the a and b register sets
            auto &wc = (j & 1) ? wfb : wfa;
            auto &xc = (j & 1) ? xfb : xfa;
            auto &wn = (j & 1) ? wfa : wfb;
            auto &xn = (j & 1) ? xfa : xfb;
            if (j + 1 < R) {
                read_frags<Cfg>(wn, xn, stage, waddr[j + 1], xaddr[j + 1]);
            } else {
                // Stage kt+1 must have landed and every wave must be done reading
                // stage kt before its slot is refilled.  In steady state S-1 stages
                // are in flight, so "at most S-2 outstanding" means kt+1 is in.
                if (STEADY)
                    __builtin_amdgcn_s_waitcnt(waitcnt_imm(L * (S - 2), 0));
                else
                    __builtin_amdgcn_s_waitcnt(waitcnt_imm(0, 0));
                lds_barrier();
                // (the LDS reads come first in program order: the compiler must assume
                // the direct-to-LDS loads may alias them and would not move reads above)
                if (STEADY || kt + 1 < ksteps) read_frags<Cfg>(wn, xn, lds + nxt * Cfg::kStageBytes, waddr[0], xaddr[0]);
            }
            widen_frags<Cfg, 1>(hi, wc, xc);
            mma_step<Cfg>(acc, lo);
            schedule_region<Cfg, Cfg::kNI + Cfg::kMI, 0>();
            if (STEADY && j + 1 == R) issue_stage<Cfg>(wsrc, xsrc, kpos(kt + S) * RB, goff, lds + cur * Cfg::kStageBytes, wave);
            widen_frags<Cfg, 0>(lo, wn, xn);
            mma_step<Cfg>(acc, hi);
            if (STEADY && j + 1 == R)
                schedule_region<Cfg, 0, Cfg::kLoads>();
            else
                schedule_region<Cfg, 0, 0>();
        }
        cur = nxt;
    };
    int kt = 0;
    for (; kt + S < ksteps; ++kt) k_step(kt, std::true_type{});
    for (; kt < ksteps; ++kt) k_step(kt, std::false_type{});

    // Epilogue.  Accumulator register r of a 32x32 tile holds
    // n = 8*(r/4) + 4*(lane/32) + r%4, m = lane%32.
    if (!ACC_OUT && out_dtype == VDMQ_OUT_F16) {
        // fp16 path: scale in the accumulator layout, round to fp16, transpose one
        // 32-row strip at a time through LDS (the stage ring is idle: every wave
        // passed the last barrier after its final LDS read and no load is in
        // flight), then add the bias and store 16 bytes per lane so that a row's
        // kWaveN outputs leave as whole 128-byte lines.
        constexpr int PR = Cfg::kPiecesPerRow, RS = Cfg::kStageRowBytes;
        uint8_t *stg = lds + wave * Cfg::kStagingBytes;
        // channel scales of this wave's columns as fp32, once per tile
        float wsf[Cfg::kNI][4][4];
#pragma unroll
        for (int ni = 0; ni < Cfg::kNI; ++ni)
#pragma unroll
            for (int rg = 0; rg < 4; ++rg) {
                const f16x4 w4 = *reinterpret_cast<const f16x4 *>(side + Cfg::kSideWs + (ni * 32 + rg * 8 + lh * 4) * 2);
#pragma unroll
                for (int e = 0; e < 4; ++e) wsf[ni][rg][e] = static_cast<float>(w4[e]);
            }
        const int ncol = n0 + wn0 + (lane % PR) * 8;
        const f16x8 bv = *reinterpret_cast<const f16x8 *>(side + Cfg::kSideBias + (lane % PR) * 16); /* -0 without a bias */
        // The stores are buffer stores: the wave's corner of the output is the resource, whose size ends with the
        // last row below M, so rows beyond are dropped by the range check instead of being predicated.  The check
        // looks at the vector offset only (a scalar offset is added after it), so the row goes into the vector
        // offset: one addition per store where a 64-bit address takes a multiplication and several additions.
        const int wave_rows = min(max(M - (m0 + wm0), 0), Cfg::kWaveM);
        if (n0 + wn0 >= N || wave_rows == 0) return; /* the same for the whole wave */
        const int part = tail.split_cols != 0 ? (n0 + wn0) / tail.split_cols : 0; /* the wave's columns lie inside one part */
        const __amdgpu_buffer_rsrc_t out_rsrc = __builtin_amdgcn_make_buffer_rsrc(
            static_cast<__half *>(out) + part * tail.part_stride + static_cast<int64_t>(m0 + wm0) * ldo + (n0 + wn0 - part * tail.split_cols), 0,
            wave_rows * static_cast<int>(ldo) * 2, 0x00020000);
        const int out_voff = ((lane / PR) * static_cast<int>(ldo) + (lane % PR) * 8) * 2;
        // Row of the gate vectors for output row m = m / rows_per_gate, without a division per element: one vector per
        // token is the row itself, and with at least as many rows per vector as the wave owns the wave's rows meet at
        // most one boundary, found by comparing with the first row's remainder.
        const int gate_rows = TAIL ? tail.rows_per_gate : 1;
        const int gate_first = __builtin_amdgcn_readfirstlane((m0 + wm0) / gate_rows), gate_rem = m0 + wm0 - gate_first * gate_rows;
        auto gate_row = [&](int mrow) -> int64_t {
            if (gate_rows == 1) return mrow;
            if (gate_rows >= Cfg::kWaveM) return gate_first + (gate_rem + (mrow - m0 - wm0) >= gate_rows ? 1 : 0);
            return mrow / gate_rows;
        };
#pragma unroll
        for (int mi = 0; mi < Cfg::kMI; ++mi) {
            // The accumulator holds 256*acc.  float(256*acc) = 256*float(acc) exactly (|acc| < 2^24),
            // and scaling the token scale by 2^-8 is exact too, so
            //   float(256*acc) * fl((as/256) * ws) == fl(float(acc) * fl(as * ws))   bit for bit
            // (no under- or overflow: as*ws/256 >= 2^-56, |256*acc| < 2^31).
            const float as = static_cast<float>(*reinterpret_cast<const _Float16 *>(side + Cfg::kSideAs + (mi * 32 + l32) * 2)) * 0.00390625f;
            // gate and residual pieces of this strip, requested before the strip is converted and
            // staged so that their latency runs under that work
            f16x8 gv[PR / 2], rv[PR / 2];
#pragma unroll
            for (int it = 0; TAIL && it < PR / 2; ++it) {
                const int mrow = m0 + wm0 + mi * 32 + it * (64 / PR) + lane / PR;
                const bool live = mrow < M && ncol < N;
                if (tail.gate != nullptr && live)
                    gv[it] = *reinterpret_cast<const f16x8 *>(tail.gate + gate_row(mrow) * tail.ldg + ncol);
                if (tail.residual != nullptr && live)
                    rv[it] = *reinterpret_cast<const f16x8 *>(tail.residual + static_cast<int64_t>(mrow) * tail.ldr + ncol);
            }
#pragma unroll
            for (int ni = 0; ni < Cfg::kNI; ++ni)
#pragma unroll
                for (int rg = 0; rg < 4; ++rg) {
                    f16x4 h;
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const float v = static_cast<float>(acc[ni][mi][rg * 4 + e]) * (as * wsf[ni][rg][e]);
                        h[e] = static_cast<_Float16>(v); /* round to nearest even */
                    }
                    *reinterpret_cast<f16x4 *>(stg + l32 * RS + (ni * 32 + rg * 8 + lh * 4) * 2) = h;
                }
#pragma unroll
            for (int it = 0; it < PR / 2; ++it) {
                const int row = it * (64 / PR) + lane / PR;
                f16x8 hv = *reinterpret_cast<const f16x8 *>(stg + row * RS + (lane % PR) * 16);
                hv += bv; /* one fp16 add per element */
                const int mrow = m0 + wm0 + mi * 32 + row;
                // out = residual + y * gate: the block's gated residual update, two more fp16
                // operations per element, each rounded like the fp16 tensor operations they replace
                if (TAIL && tail.gate != nullptr && mrow < M) hv *= gv[it];
                if (TAIL && tail.residual != nullptr && mrow < M) hv = rv[it] + hv;
                // A large output is not re-read before it falls out of the caches anyway: streaming it (nt) keeps
                // the operands (and the next quantizer's writes) in the Infinity Cache (measured: next quantizer
                // 5.76 -> 6.01 TB/s).
                __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, hv), out_rsrc,
                                                       out_voff + (mi * 32 + it * (64 / PR)) * static_cast<int>(ldo) * 2, 0,
                                                       STREAM_OUT ? 2 /* nt */ : 0);
            }
        }
        return;
    }
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
                    // bf16 output (not offered by the reference): same fp32 product, the
                    // fp16 bias added in fp32, one rounding to bf16.
                    const f16x4 ws = *reinterpret_cast<const f16x4 *>(wscale + n);
                    uint32_t o[2];
#pragma unroll
                    for (int e2 = 0; e2 < 2; ++e2) {
                        uint32_t pk = 0;
#pragma unroll
                        for (int e = 0; e < 2; ++e) {
                            float f = static_cast<float>(acc[ni][mi][rg * 4 + 2 * e2 + e] >> 8) * (as * static_cast<float>(ws[2 * e2 + e]));
                            if (bias != nullptr) f += static_cast<float>(reinterpret_cast<const _Float16 *>(bias)[n + 2 * e2 + e]);
                            uint32_t u = __float_as_uint(f);
                            u = (f != f) ? 0x7FC00000u : u + 0x7FFFu + ((u >> 16) & 1u); /* RNE */
                            pk |= (u >> 16) << (16 * e);
                        }
                        o[e2] = pk;
                    }
                    typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));
                    u32x2 ov = {o[0], o[1]};
                    *reinterpret_cast<u32x2 *>(static_cast<uint16_t *>(out) + static_cast<int64_t>(m) * ldo + n) = ov;
                }
            }
        }
    }
#endif
}

template <typename Cfg>
int launch_cfg(const uint8_t *qact, const __half *ascale, const uint8_t *wq, const __half *wscale, const __half *bias, void *out,
               int out_dtype, int32_t *acc_out, int64_t M, int64_t N, int64_t K, int64_t ldo, const GemmTail &tail, hipStream_t s) {
    TileMap tm;
    tm.tiles_m = static_cast<int>(ceil_div(M, Cfg::BM));
    tm.tiles_n = static_cast<int>(ceil_div(N, Cfg::BN));
    const int super_m = static_cast<int>(ceil_div(tm.tiles_m, kGroupM));
    tm.super_n = static_cast<int>(ceil_div(tm.tiles_n, kGroupN));
    const int64_t total_super = static_cast<int64_t>(super_m) * tm.super_n;
    if (total_super * kGroupM * kGroupN + kXcds * kGroupM * kGroupN > (int64_t(1) << 30))
        return fail(VDMQ_ESHAPE, "M x N = %lld x %lld needs more workgroups than one launch can hold", (long long)M, (long long)N);
    // Split the super-tile sequence (n fastest) into kXcds runs of equal tile counts.  tiles_before(st)
    // is monotone, so each boundary is a binary search.
    const int64_t last_m = tm.tiles_m - static_cast<int64_t>(super_m - 1) * kGroupM; /* tile rows of the last super-row */
    auto tiles_before = [&](int64_t st) {
        const int64_t sm = st / tm.super_n, sn = st % tm.super_n;
        const int64_t rows_here = sm == super_m - 1 ? last_m : kGroupM;
        const int64_t cols_done = sn * kGroupN < tm.tiles_n ? sn * kGroupN : tm.tiles_n;
        return sm * kGroupM * tm.tiles_n + rows_here * cols_done;
    };
    const int64_t all_tiles = static_cast<int64_t>(tm.tiles_m) * tm.tiles_n;
    tm.start[0] = 0;
    int rounds = 0;
    for (int x = 1; x <= kXcds; ++x) {
        const int64_t want = (all_tiles * x + kXcds - 1) / kXcds;
        int64_t lo = tm.start[x - 1], hi = total_super; /* first st with tiles_before(st) >= want */
        while (lo < hi) {
            const int64_t mid = (lo + hi) / 2;
            if (tiles_before(mid) >= want) hi = mid; else lo = mid + 1;
        }
        tm.start[x] = x == kXcds ? static_cast<int>(total_super) : static_cast<int>(lo);
        rounds = rounds > tm.start[x] - tm.start[x - 1] ? rounds : tm.start[x] - tm.start[x - 1];
    }
    // measured: the contiguous order wins with one workgroup per CU and K >= 3072 (+1 %, 18 % less traffic
    // beyond L2), loses with two workgroups per CU (-3 %) and at K = 1536 (-4 %)
    tm.contig = Cfg::kOccupancy == 1 && K >= 2048;
    if (!tm.contig) rounds = static_cast<int>(ceil_div(total_super, kXcds));
    const dim3 grid(static_cast<unsigned>(rounds) * kXcds * kGroupM * kGroupN), block(Cfg::kThreads);
    const int ldk = static_cast<int>(k_padded(K) / 2);

    // A large output is not re-read before it falls out of the caches anyway:
    // streaming it keeps the operands (and the next quantizer's writes) in the
    // Infinity Cache.
    const bool stream_out = M * N * 2 > (int64_t(224) << 20);
    const bool has_tail = tail.gate != nullptr || tail.residual != nullptr;
    const int which = acc_out != nullptr ? 2 : (stream_out ? 1 : 0) + (has_tail ? 3 : 0);
    using Kernel = void (*)(const uint8_t *, const uint8_t *, const __half *, const __half *, const __half *, void *, int, int32_t *, int,
                            int, int, int64_t, TileMap, GemmTail);
    const Kernel kernels[5] = {gemm_w4a4_kernel<Cfg, 0>, gemm_w4a4_kernel<Cfg, 1>, gemm_w4a4_kernel<Cfg, 2>, gemm_w4a4_kernel<Cfg, 3>,
                               gemm_w4a4_kernel<Cfg, 4>};
    // LDS above 64 KiB has to be requested once per kernel and device
    constexpr int kMaxDevices = 64;
    static bool attr_done[kMaxDevices][5] = {};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return fail(VDMQ_ELAUNCH, "no current HIP device");
    if (!attr_done[dev][which]) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kernels[which]), hipFuncAttributeMaxDynamicSharedMemorySize,
                                           Cfg::kLdsBytes);
        if (e != hipSuccess) return fail(VDMQ_ELAUNCH, "hipFuncSetAttribute(%d bytes of LDS): %s", Cfg::kLdsBytes, hipGetErrorString(e));
        attr_done[dev][which] = true;
    }
    hipLaunchKernelGGL(kernels[which], grid, block, Cfg::kLdsBytes, s, qact, wq, ascale, wscale, bias, out, out_dtype, acc_out,
                       static_cast<int>(M), static_cast<int>(N), ldk, ldo, tm, tail);
    const int rc = check_launch("gemm_w4a4_kernel");
    if (rc == VDMQ_OK) record_gemm_launch({VDMQ_KERNEL_GEMM_W4A4, Cfg::BM, Cfg::BN, kGroupM, kGroupN, tm.contig, static_cast<int64_t>(grid.x)});
    return rc;
}

}  // namespace

int launch_gemm(const uint8_t *qact, const __half *ascale, const uint8_t *wq, const __half *wscale, const __half *bias, void *out,
                int out_dtype, int32_t *acc_out, int64_t M, int64_t N, int64_t K, int64_t ldo, const GemmTail &tail, hipStream_t s) {
    if (M == 0 || N == 0) return VDMQ_OK;
    // One 8-wave workgroup per CU with a 256 x 256 tile is the fastest steady state, but its
    // prologue and epilogue run with the matrix pipes idle.  When a CU sees only a few such
    // tiles, or K is short, two 4-wave workgroups per CU (one's epilogue under the other's K
    // loop) win: 256 x 128 tiles (Wan-1.3B: o-proj +19 %, FFN-down +12 %, QKV +4 %).  With
    // fewer than two large tiles per CU (M = 512 text tokens) 128 x 128 tiles fill the chip.
    using Big = GemmCfg<256, 256, 2, 4, 2, 1, 256>;
    using Mid = GemmCfg<256, 128, 2, 2, 3, 2, 128>;
    using Small = GemmCfg<128, 128, 2, 2, 3, 2, 128>;
    const int64_t big_tiles = ceil_div(M, Big::BM) * ceil_div(N, Big::BN);
    if (big_tiles < 512) return launch_cfg<Small>(qact, ascale, wq, wscale, bias, out, out_dtype, acc_out, M, N, K, ldo, tail, s);
    if (big_tiles < 1024 || (K < 2048 && big_tiles < 4096))
        return launch_cfg<Mid>(qact, ascale, wq, wscale, bias, out, out_dtype, acc_out, M, N, K, ldo, tail, s);
    return launch_cfg<Big>(qact, ascale, wq, wscale, bias, out, out_dtype, acc_out, M, N, K, ldo, tail, s);
}

}  // namespace vdmq
