// W8A8 int8 and FP8 (OCP e4m3fn / e5m2) GEMMs on the gfx950 matrix cores.
//
//   acc[m,n] = sum_k A[m,k] * B[n,k]        A: [M,K] row-major, B: [N,K] row-major
//
// Both operands are K-contiguous, which is exactly what an MFMA lane wants (each lane feeds
// 16 or 32 consecutive K-bytes of one row), so tiles move global -> LDS -> registers as
// 16-byte chunks and nothing is ever transposed.
//
// Kernel shape (template GemmCfg): a block of WM x WN wavefronts owns a BM x BN output tile
// and walks K in BK-byte steps through a double-buffered LDS ring; each wavefront owns a
// (BM/WM) x (BN/WN) sub-tile made of 32x32 MFMA tiles:
//   int8: v_mfma_i32_32x32x32_i8      (16 K-bytes per lane per operand, 8 passes)
//   fp8 : v_mfma_f32_32x32x64_f8f6f4  (32 K-bytes per lane per operand, 16 passes; the
//         legacy v_mfma_f32_32x32x16_fp8_fp8 runs at half that rate on gfx950)
// LDS rows are BK bytes; the 16-byte chunk index is XOR-swizzled with the row so that the
// ds_read_b128 of 16 consecutive rows hits every bank exactly once.
// The flat block id is first remapped so that each of the 8 XCDs (private L2 each) gets a
// contiguous range of tiles, then walked in groups of GROUP_M tile-rows for L2 reuse.
// Split-K (gridDim.y > 1) writes raw accumulators to a workspace; a second kernel reduces
// them in a fixed order (deterministic) and applies the epilogue.
#pragma once
#include <algorithm>
#include <type_traits>

#include "gemm_tile.h"
#include "llmq_common.h"

#ifndef LLMQ_LDS_EPILOGUE
#define LLMQ_LDS_EPILOGUE 1
#endif

namespace llmq {
namespace {


typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));

constexpr int kNumXcd = 8;
constexpr int kGroupM = 8;


__device__ __forceinline__ uint16_t to_out(float v, int out_dtype) {
    return out_dtype == LLMQ_BF16 ? Lo<LLMQ_BF16>::from_f32(v) : Lo<LLMQ_F16>::from_f32(v);
}

template <int BM_, int BN_, int BK_, int WM_, int WN_, bool FP8_, int AFMT_ = 0, int RS_ = 2, bool DMA_ = false>
struct GemmCfg {
    static constexpr int BM = BM_, BN = BN_, BK = BK_, WM = WM_, WN = WN_;
    static constexpr int RS = RS_;                     // K tiles staged in registers: 2, or 1 for fat tiles
    static constexpr bool FP8 = FP8_;
    static constexpr int AFMT = AFMT_;                 // fp8 A format selector: 0 e4m3, 1 e5m2; without FP8: 2 = fp16 operands
    static constexpr bool F16 = !FP8_ && AFMT_ == 2;   // v_mfma_f32_32x32x16_f16: 16 K-elements = 32 K-bytes per MFMA, like int8
    static constexpr bool FACC = FP8_ || F16;          // fp32 accumulators
    static constexpr int NT = WM * WN * kWave;
    static constexpr int WTM = BM / WM, WTN = BN / WN; // wavefront tile
    static constexpr int TM = WTM / 32, TN = WTN / 32; // MFMA tiles per wavefront
    static constexpr int CPR = BK / 16;                // 16-byte chunks per LDS row
    static constexpr int ROWS_PER_LINE = 16 / CPR;     // rows per 256-byte bank line
    static constexpr int KB = FP8 ? 64 : 32;           // K-bytes one MFMA consumes
    static constexpr int KSUB = BK / KB;
    static constexpr int A_LOADS = BM * CPR / NT, B_LOADS = BN * CPR / NT;
    static constexpr int STAGE_CHUNKS = (BM + BN) * CPR;
    static constexpr bool DMA = DMA_;                  // operand tiles go global -> LDS directly (global_load_lds), as many LDS stages as fit (up to 4)
    static constexpr int STAGES = !DMA ? 2 : (4 * STAGE_CHUNKS * 16 <= 160 * 1024 ? (STAGE_CHUNKS * 16 <= 24 * 1024 && BK == 128 ? 3 : 4)
                                                                                   : (3 * STAGE_CHUNKS * 16 <= 160 * 1024 ? 3 : 2));
    static constexpr size_t LDS_BYTES = (size_t)STAGES * STAGE_CHUNKS * 16u;
    // Double-buffer the MFMA operand fragments (software pipeline LDS reads under MFMAs).  The fp8
    // fragments are twice as wide; with two wavefronts per SIMD (256 registers each) they do not fit twice.
    static constexpr bool PIPE = DMA || (!(FP8 && NT > 256) && !(RS == 1 && NT > 256));
    static_assert(BM % (WM * 32) == 0 && BN % (WN * 32) == 0, "wave tile must be 32-aligned");
    static_assert((BM * CPR) % NT == 0 && (BN * CPR) % NT == 0, "tile must split evenly over threads");
    static_assert(CPR == 4 || CPR == 8, "BK must be 64 or 128");
};

template <int CPR>
__device__ __forceinline__ int lds_chunk(int row, int c) {
    return row * CPR + (c ^ ((row / (16 / CPR)) & (CPR - 1)));
}

// flat block id -> (tile_m, tile_n): XCD-contiguous ranges, then GROUP_M-row swizzle
__device__ __forceinline__ void tile_coords(int bid, int nblk, int tiles_m, int tiles_n, int& tm, int& tn) {
    const int q = nblk / kNumXcd, r = nblk % kNumXcd;
    const int xcd = bid % kNumXcd, local = bid / kNumXcd;
    const int pid = xcd < r ? xcd * (q + 1) + local : r * (q + 1) + (xcd - r) * q + local;
    const int width = kGroupM * tiles_n;
    const int group = pid / width, first_m = group * kGroupM;
    const int gsize = min(tiles_m - first_m, kGroupM);
    tm = first_m + (pid % width) % gsize;
    tn = (pid % width) / gsize;
}

template <class C, bool KFULL>
__global__ __launch_bounds__(C::NT) void gemm_tile_kernel(
    const uint8_t* __restrict__ A, int64_t lda, const uint8_t* __restrict__ B, int64_t ldb,
    int M, int N, int K, int k_per_split, Epilogue ep, void* __restrict__ out, int64_t ldo,
    void* __restrict__ acc_dump, void* __restrict__ partials) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem_raw[];
    uint4* lds = reinterpret_cast<uint4*>(smem_raw);
    using acc_t = typename std::conditional<C::FACC, v16f, v16i>::type;

    const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
    const int wm = wave / C::WN, wn = wave % C::WN;
    const int tiles_m = (M + C::BM - 1) / C::BM, tiles_n = (N + C::BN - 1) / C::BN;
    int tile_m, tile_n;
    tile_coords(blockIdx.x, gridDim.x, tiles_m, tiles_n, tile_m, tile_n);
    const int m0 = tile_m * C::BM, n0 = tile_n * C::BN;
    const int k_begin = blockIdx.y * k_per_split;
    const int k_end = min(K, k_begin + k_per_split);
    const int ktiles = (k_end - k_begin + C::BK - 1) / C::BK;

    // ---- global -> register staging.  Slot i of a thread is row (tid / CPR) + i * ROWS_STEP at
    // chunk tid % CPR: the chunk (hence the LDS swizzle) is the same for all of a thread's slots.
    constexpr int ROWS_STEP = C::NT / C::CPR;
    static_assert(ROWS_STEP % 16 == 0, "row step must keep the swizzle phase");
    const int ld_row = tid / C::CPR, ld_c = tid % C::CPR;
    const uint8_t* a_base = A + (int64_t)m0 * lda + k_begin + ld_c * 16;
    const uint8_t* b_base = B + (int64_t)n0 * ldb + k_begin + ld_c * 16;
    int a_off[C::A_LOADS], b_off[C::B_LOADS];  // byte offsets of the (clamped) rows inside the tile
#pragma unroll
    for (int i = 0; i < C::A_LOADS; i++) a_off[i] = min(ld_row + i * ROWS_STEP, M - 1 - m0) * (int)lda;
#pragma unroll
    for (int i = 0; i < C::B_LOADS; i++) b_off[i] = min(ld_row + i * ROWS_STEP, N - 1 - n0) * (int)ldb;
    const int st_a = lds_chunk<C::CPR>(ld_row, ld_c);
    const int st_b = C::BM * C::CPR + st_a;
    uint4 ra[C::RS][C::A_LOADS], rb[C::RS][C::B_LOADS];  // tiles in flight (register staging)
    // Loads are unconditional (branch-free), so the compiler can count them and wait for exactly the
    // tile it is about to store while younger loads stay in flight.  A tile index past the end of this
    // split's K range re-reads the last tile, a chunk past the ragged end of K re-reads chunk 0 of its
    // row; both are replaced by zeros when the tile is stored to LDS (the main loop always runs an even
    // number of tiles).
    auto load_tile = [&](int kt, uint4* a_reg, uint4* b_reg) {
        int koff = max(min(kt, ktiles - 1), 0) * C::BK;
        if constexpr (!KFULL) koff -= (ld_c * 16 < k_end - k_begin - koff) ? 0 : ld_c * 16;
#pragma unroll
        for (int i = 0; i < C::A_LOADS; i++) a_reg[i] = *reinterpret_cast<const uint4*>(a_base + a_off[i] + koff);
#pragma unroll
        for (int i = 0; i < C::B_LOADS; i++) b_reg[i] = *reinterpret_cast<const uint4*>(b_base + b_off[i] + koff);
    };
    auto store_tile = [&](int stage, int kt, const uint4* a_reg, const uint4* b_reg) {
        uint4* s = lds + stage * C::STAGE_CHUNKS;
        const bool ok = kt < ktiles && (KFULL || ld_c * 16 < k_end - k_begin - kt * C::BK);
        const uint32_t keep = ok ? 0xffffffffu : 0u;
#pragma unroll
        for (int i = 0; i < C::A_LOADS; i++) {
            const uint4 v = a_reg[i];
            s[st_a + i * ROWS_STEP * C::CPR] = make_uint4(v.x & keep, v.y & keep, v.z & keep, v.w & keep);
        }
#pragma unroll
        for (int i = 0; i < C::B_LOADS; i++) {
            const uint4 v = b_reg[i];
            s[st_b + i * ROWS_STEP * C::CPR] = make_uint4(v.x & keep, v.y & keep, v.z & keep, v.w & keep);
        }
    };
    // Block barrier that orders LDS traffic only: global loads stay in flight across it.
    auto lds_barrier = [] {
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
    };

    acc_t acc[C::TM][C::TN];
#pragma unroll
    for (int i = 0; i < C::TM; i++)
#pragma unroll
        for (int j = 0; j < C::TN; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0;

    // ---- LDS -> MFMA operand addressing -----------------------------------------------------
    const int l32 = lane & 31, khalf = lane >> 5;  // row within the 32-row tile, K half of the lane
    const int a_row0 = wm * C::WTM + l32, b_row0 = wn * C::WTN + l32;

    // MFMA operand fragments, double-buffered: while the matrix pipe works on one K sub-step the LDS
    // already serves the reads of the next one (also across the block barrier, so the first reads of a
    // freshly published stage overlap the last MFMAs of the previous tile).
    using frag_t = typename std::conditional<C::FP8, v8i, v4i>::type;
    frag_t fa[C::PIPE ? 2 : 1][C::TM], fb[C::PIPE ? 2 : 1][C::TN];
    auto read_frags = [&](int stage, int ks, frag_t* af, frag_t* bf) {
        const uint4* sA = lds + stage * C::STAGE_CHUNKS;
        const uint4* sB = sA + C::BM * C::CPR;
        if constexpr (C::FP8) {
            const int c0 = ks * 4 + khalf * 2;
#pragma unroll
            for (int i = 0; i < C::TM; i++) {
                const int row = a_row0 + i * 32;
                const uint4 lo = sA[lds_chunk<C::CPR>(row, c0)], hi = sA[lds_chunk<C::CPR>(row, c0 + 1)];
                af[i] = v8i{(int)lo.x, (int)lo.y, (int)lo.z, (int)lo.w, (int)hi.x, (int)hi.y, (int)hi.z, (int)hi.w};
            }
#pragma unroll
            for (int j = 0; j < C::TN; j++) {
                const int row = b_row0 + j * 32;
                const uint4 lo = sB[lds_chunk<C::CPR>(row, c0)], hi = sB[lds_chunk<C::CPR>(row, c0 + 1)];
                bf[j] = v8i{(int)lo.x, (int)lo.y, (int)lo.z, (int)lo.w, (int)hi.x, (int)hi.y, (int)hi.z, (int)hi.w};
            }
        } else {
            const int c0 = ks * 2 + khalf;
#pragma unroll
            for (int i = 0; i < C::TM; i++) {
                const uint4 v = sA[lds_chunk<C::CPR>(a_row0 + i * 32, c0)];
                af[i] = v4i{(int)v.x, (int)v.y, (int)v.z, (int)v.w};
            }
#pragma unroll
            for (int j = 0; j < C::TN; j++) {
                const uint4 v = sB[lds_chunk<C::CPR>(b_row0 + j * 32, c0)];
                bf[j] = v4i{(int)v.x, (int)v.y, (int)v.z, (int)v.w};
            }
        }
    };
    auto mfma_step = [&](const frag_t* af, const frag_t* bf) {
#pragma unroll
        for (int i = 0; i < C::TM; i++)
#pragma unroll
            for (int j = 0; j < C::TN; j++) {
                if constexpr (C::FP8)
                    acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(bf[j], af[i], acc[i][j], 0, C::AFMT,
                                                                                0, 0, 0, 0);
                else if constexpr (C::F16)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(v8h, bf[j]), __builtin_bit_cast(v8h, af[i]),
                                                                       acc[i][j], 0, 0, 0);
                else
                    acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(bf[j], af[i], acc[i][j], 0, 0, 0);
            }
    };
    // Scheduling directive for one sub-step: issue the LDS reads of the next fragments one by one
    // between the MFMAs of the current fragments (reads first), instead of after them.
    auto interleave_reads_with_mfma = [] {
        constexpr int kReads = (C::TM + C::TN) * (C::FP8 ? 2 : 1), kMfma = C::TM * C::TN;
        constexpr int kPairs = kReads < kMfma ? kReads : kMfma;
#pragma unroll
        for (int n = 0; n < kPairs; n++) {
            __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);  // one DS read
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);  // one MFMA
        }
        if (kReads > kPairs) __builtin_amdgcn_sched_group_barrier(0x100, kReads - kPairs, 0);
        if (kMfma > kPairs) __builtin_amdgcn_sched_group_barrier(0x008, kMfma - kPairs, 0);
    };
    // Same for the first sub-step of a tile, which also carries the LDS writes of the next tile: reads
    // first (one per MFMA), then the writes spread over the remaining MFMAs.
    auto interleave_reads_writes_with_mfma = [] {
        constexpr int kReads = (C::TM + C::TN) * (C::FP8 ? 2 : 1), kMfma = C::TM * C::TN;
        constexpr int kWrites = C::A_LOADS + C::B_LOADS;
        constexpr int kPairs = kReads < kMfma ? kReads : kMfma;
#pragma unroll
        for (int n = 0; n < kPairs; n++) {
            __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        }
        if (kReads > kPairs) __builtin_amdgcn_sched_group_barrier(0x100, kReads - kPairs, 0);
        constexpr int kRest = kMfma - kPairs;
        if constexpr (kRest > 0) {
            constexpr int kPer = (kWrites + kRest - 1) / kRest;
#pragma unroll
            for (int n = 0; n < kRest; n++) {
#pragma unroll
                for (int w = 0; w < kPer; w++)
                    if (n * kPer + w < kWrites) __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);  // one DS write
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            }
        } else {
            __builtin_amdgcn_sched_group_barrier(0x200, kWrites, 0);
        }
    };
    // One K tile.  With two or more sub-steps the next tile (registers -> other stage; nobody reads that
    // stage any more once the previous tile's barrier is passed) is written to LDS under the MFMAs of
    // sub-step 0; sub-steps 0 .. KSUB-2 read the next sub-step of the same stage; before the last
    // sub-step the barrier publishes the other stage, whose first sub-step is read under the last MFMAs.
    // `par` is the fragment-buffer parity on entry (compile-time).
    auto tile_steps = [&](int stage, auto par_c, int kt_next, uint4* a_reg, uint4* b_reg) {
        constexpr int par = decltype(par_c)::value;
        if constexpr (!C::PIPE) {
#pragma unroll
            for (int ks = 0; ks < C::KSUB; ks++) {
                read_frags(stage, ks, fa[0], fb[0]);
                mfma_step(fa[0], fb[0]);
            }
            store_tile(stage ^ 1, kt_next, a_reg, b_reg);
            if constexpr (C::RS == 1) load_tile(kt_next + 1, a_reg, b_reg);
            lds_barrier();
        } else {
#pragma unroll
            for (int ks = 0; ks < C::KSUB - 1; ks++) {
                read_frags(stage, ks + 1, fa[(par + ks + 1) & 1], fb[(par + ks + 1) & 1]);
                if (C::RS == 2 && ks == 0) store_tile(stage ^ 1, kt_next, a_reg, b_reg);
                mfma_step(fa[(par + ks) & 1], fb[(par + ks) & 1]);
                if (C::RS == 2 && ks == 0) interleave_reads_writes_with_mfma();
                else interleave_reads_with_mfma();
                __builtin_amdgcn_sched_barrier(0);
            }
            if constexpr (C::KSUB == 1 || C::RS == 1) store_tile(stage ^ 1, kt_next, a_reg, b_reg);
            if constexpr (C::RS == 1) load_tile(kt_next + 1, a_reg, b_reg);  // refill the single register stage
            lds_barrier();
            read_frags(stage ^ 1, 0, fa[(par + C::KSUB) & 1], fb[(par + C::KSUB) & 1]);
            mfma_step(fa[(par + C::KSUB - 1) & 1], fb[(par + C::KSUB - 1) & 1]);
            interleave_reads_with_mfma();
            __builtin_amdgcn_sched_barrier(0);
        }
    };

    // ---- main loop: tile kt is computed from LDS stage kt & 1 while tile kt+1 sits in registers
    // and tile kt+2 is in flight from global memory.  Two tiles per iteration, no conditional
    // compute: an odd tile count is padded with a zero tile -----------------------------------
    if constexpr (C::DMA) {
        // Operand tiles travel global -> LDS without passing through registers (global_load_lds_dwordx4: each lane
        // names its own 16 global bytes, a wavefront's 64 pieces land back to back in LDS).  The LDS position is
        // therefore fixed by the lane and the swizzle is applied on the fetch side: the thread whose piece lands in
        // chunk slot c' of row r fetches global chunk c' ^ swizzle(r).  With NS LDS stages tile kt is computed while
        // kt+1 .. kt+NS-1 are in flight; every wait is a counted s_waitcnt on the wavefront's own loads, followed by
        // the block barrier that publishes the stage.  The loads are issued from assembly so that the compiler,
        // which would wait for every outstanding load before any later LDS read, does not see them.
        static_assert(C::KSUB % 2 == 0 && C::KSUB >= 2, "fragment parity must return to 0 at every tile");
        static_assert(KFULL, "the direct loads cannot zero a ragged K tail");
        constexpr int LPT = C::A_LOADS + C::B_LOADS;  // loads per thread and tile
        const int swz = (ld_row / (16 / C::CPR)) & (C::CPR - 1);
        const uint8_t* pa[C::A_LOADS];
        const uint8_t* pb[C::B_LOADS];
#pragma unroll
        for (int i = 0; i < C::A_LOADS; i++) pa[i] = A + (int64_t)m0 * lda + k_begin + a_off[i] + (ld_c ^ swz) * 16;
#pragma unroll
        for (int i = 0; i < C::B_LOADS; i++) pb[i] = B + (int64_t)n0 * ldb + k_begin + b_off[i] + (ld_c ^ swz) * 16;
        const uint32_t lds_base = (uint32_t)(uintptr_t)((__attribute__((address_space(3))) void*)smem_raw);
        const uint32_t wave_off = (uint32_t)__builtin_amdgcn_readfirstlane(wave) * 1024u;
        // int32 accumulators (any summation order gives the same bits): every XCD starts its walk over K at another
        // eighth and wraps around (blockIdx.x % 8 is the XCD), so the eight L2s ask the fabric for different lines of the
        // shared panels at any moment instead of all for the same ones.  The blocks of one XCD stay in step, which is what
        // lets them share a panel through their L2.  fp32 accumulators keep the natural order: their bits would
        // otherwise depend on where in the grid a tile sits.
        const int krot = C::FACC ? 0 : (int)((blockIdx.x % kNumXcd) * (unsigned)ktiles / kNumXcd);
        auto issue_tile = [&](int kt, int stage) {
            int kr = min(kt, ktiles - 1) + krot;  // past the end: the last tile again, into a stage nobody reads
            kr -= kr >= ktiles ? ktiles : 0;
            const int koff = kr * C::BK;
            const uint32_t sbase = lds_base + (uint32_t)stage * (C::STAGE_CHUNKS * 16u) + wave_off;
#pragma unroll
            for (int i = 0; i < C::A_LOADS; i++) {
                const uint32_t m0v = sbase + (uint32_t)i * (C::NT * 16u);
                asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(m0v), "v"(pa[i] + koff) : "memory", "m0");
            }
#pragma unroll
            for (int i = 0; i < C::B_LOADS; i++) {
                const uint32_t m0v = sbase + (uint32_t)(C::BM * C::CPR * 16) + (uint32_t)i * (C::NT * 16u);
                asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(m0v), "v"(pb[i] + koff) : "memory", "m0");
            }
        };
        constexpr int NS = C::STAGES;
        auto wait_next_tile = [] {  // at most the NS - 2 youngest tiles may still be in flight
            constexpr int N = (NS - 2) * LPT;
            static_assert(N < 64, "vmcnt is a 6-bit counter");
            asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
        };
#pragma unroll
        for (int t = 0; t < NS - 1; t++) issue_tile(t, t);
        wait_next_tile();
        lds_barrier();
        read_frags(0, 0, fa[0], fb[0]);
        int stage = 0;
#pragma unroll 1
        for (int kt = 0; kt < ktiles; kt++) {
            const int prev = stage == 0 ? NS - 1 : stage - 1, next = stage == NS - 1 ? 0 : stage + 1;
            issue_tile(kt + NS - 1, prev);  // the stage of tile kt-1: every wavefront passed the last barrier after reading it
#pragma unroll
            for (int ks = 0; ks < C::KSUB - 1; ks++) {
                read_frags(stage, ks + 1, fa[(ks + 1) & 1], fb[(ks + 1) & 1]);
                mfma_step(fa[ks & 1], fb[ks & 1]);
                interleave_reads_with_mfma();
                __builtin_amdgcn_sched_barrier(0);
            }
            wait_next_tile();  // tile kt+1 has landed
            lds_barrier();
            read_frags(next, 0, fa[0], fb[0]);
            mfma_step(fa[(C::KSUB - 1) & 1], fb[(C::KSUB - 1) & 1]);
            interleave_reads_with_mfma();
            __builtin_amdgcn_sched_barrier(0);
            stage = next;
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // nothing may still be landing in LDS when it is reused or released
        lds_barrier();
    } else if constexpr (C::RS == 2) {
        load_tile(0, ra[0], rb[0]);
        load_tile(1, ra[1], rb[1]);
        store_tile(0, 0, ra[0], rb[0]);
        lds_barrier();
        if constexpr (C::PIPE) read_frags(0, 0, fa[0], fb[0]);
#pragma unroll 1
        for (int kt = 0; kt < ktiles; kt += 2) {
            load_tile(kt + 2, ra[0], rb[0]);
            tile_steps(0, std::integral_constant<int, 0>{}, kt + 1, ra[1], rb[1]);
            load_tile(kt + 3, ra[1], rb[1]);
            tile_steps(1, std::integral_constant<int, C::KSUB & 1>{}, kt + 2, ra[0], rb[0]);
        }
    } else {
        // fat tiles: one register stage; tile kt+1 is stored late in tile kt and the stage is refilled
        // with tile kt+2 right away, which then has a whole tile time to arrive
        load_tile(0, ra[0], rb[0]);
        store_tile(0, 0, ra[0], rb[0]);
        load_tile(1, ra[0], rb[0]);
        lds_barrier();
        if constexpr (C::PIPE) read_frags(0, 0, fa[0], fb[0]);
#pragma unroll 1
        for (int kt = 0; kt < ktiles; kt += 2) {
            tile_steps(0, std::integral_constant<int, 0>{}, kt + 1, ra[0], rb[0]);
            tile_steps(1, std::integral_constant<int, C::KSUB & 1>{}, kt + 2, ra[0], rb[0]);
        }
    }

    // ---- epilogue.  The weights feed the MFMA row operand, so D is the transposed tile: a lane holds
    // token m = l32 and, in register r, channel 8*(r/4) + 4*khalf + r%4 -> 4 consecutive channels per
    // register quad.  After the dequant math the two half-waves exchange quads (v_permlane32_swap) so
    // that every lane owns 8 consecutive channels of its token and stores them as one 16-byte vector,
    // the two lanes of a token adjacent to each other.
    const bool split = gridDim.y > 1;
    const float alpha = ep.alpha * (ep.alpha_dev ? *ep.alpha_dev : 1.0f);
    const bool out_vec = ((ldo & 7) == 0) && ((reinterpret_cast<uintptr_t>(out) & 15u) == 0);
    const bool raw_vec = (N & 3) == 0;
    const bool plain = !ep.bias && alpha == 1.0f;  // block-uniform
    const float out_scale = ep.out_scale ? *ep.out_scale : 1.0f;

    // Fast path (block-uniform): interior tile, fused epilogue, vector stores.  No per-element dtype
    // switches or bounds checks: ~5 VALU operations per output instead of several times that.
    if (!split && !acc_dump && !ep.out_scale && out_vec && m0 + C::BM <= M && n0 + C::BN <= N &&
        (reinterpret_cast<uintptr_t>(ep.w_scale) & 15u) == 0) {
        auto fast = [&](auto out_dt_c, auto plain_c) {
            constexpr int ODT = decltype(out_dt_c)::value;
            constexpr bool PLAIN = decltype(plain_c)::value;  // no bias term and alpha = 1: the scaled accumulator is the output
            // Wave tiles of 64 channels: transpose through LDS (8 KB per wavefront, 64 token rows at a time) so
            // that a store instruction writes 8 whole 128-byte rows instead of 32 pieces of 32 bytes.
            constexpr bool LDS_EPI = LLMQ_LDS_EPILOGUE && C::TM % 2 == 0 && C::TN % 2 == 0 && C::LDS_BYTES >= (C::NT / kWave) * 8192u;
            if constexpr (LDS_EPI) {
                // Every scale and bias value is fetched before the first output store is issued: loads and stores
                // share one wait counter, so a load issued after a store can only be waited for together with that
                // store's completion (microseconds when every CU writes at once).
                float sa_r[C::TM], sw_r[C::TN][16], bb_r[C::TN][16];
#pragma unroll
                for (int i = 0; i < C::TM; i++) sa_r[i] = ep.a_scale ? ep.a_scale[m0 + wm * C::WTM + i * 32 + l32] : 1.f;
#pragma unroll
                for (int j = 0; j < C::TN; j++)
#pragma unroll
                    for (int g = 0; g < 4; g++) {
                        const int n = n0 + wn * C::WTN + j * 32 + 8 * g + 4 * khalf;
                        if (ep.w_scale) {
                            const float4 v = *reinterpret_cast<const float4*>(ep.w_scale + n);
                            sw_r[j][4 * g] = v.x, sw_r[j][4 * g + 1] = v.y, sw_r[j][4 * g + 2] = v.z, sw_r[j][4 * g + 3] = v.w;
                        } else {
                            sw_r[j][4 * g] = sw_r[j][4 * g + 1] = sw_r[j][4 * g + 2] = sw_r[j][4 * g + 3] = 1.f;
                        }
#pragma unroll
                        for (int e = 0; e < 4; e++)
                            bb_r[j][4 * g + e] = ep.bias ? ep.beta * load_as_f32(ep.bias, ep.bias_dtype, n + e) : 0.f;
                    }
                __syncthreads();  // every wavefront is done reading the operand stages
                uint4* region = lds + wave * 512;
#pragma unroll
                for (int p = 0; p < C::TM / 2; p++) {
#pragma unroll
                  for (int jh = 0; jh < C::TN / 2; jh++) {  // 64 channels at a time
#pragma unroll
                    for (int jj = 0; jj < 2; jj++) {
                        const int j = 2 * jh + jj;
#pragma unroll
                        for (int ii = 0; ii < 2; ii++) {
                            const int i = 2 * p + ii;
                            const float sa = sa_r[i];
                            const int row = ii * 32 + l32, swz = (row >> 1) & 7;
                            uint32_t pk[4][2];
#pragma unroll
                            for (int g = 0; g < 4; g++) {
                                uint16_t h[4];
#pragma unroll
                                for (int e = 0; e < 4; e++) {
                                    const auto av = acc[i][j][4 * g + e];
                                    h[e] = Lo<ODT>::from_f32(epi_value<PLAIN>((float)av, sa, sw_r[j][4 * g + e], alpha, bb_r[j][4 * g + e]));
                                }
                                pk[g][0] = (uint32_t)h[0] | ((uint32_t)h[1] << 16);
                                pk[g][1] = (uint32_t)h[2] | ((uint32_t)h[3] << 16);
                            }
#pragma unroll
                            for (int g = 0; g < 2; g++) {
#pragma unroll
                                for (int x = 0; x < 2; x++) {
                                    const auto sw2 = __builtin_amdgcn_permlane32_swap(pk[2 * g][x], pk[2 * g + 1][x], false, false);
                                    pk[2 * g][x] = sw2[0];
                                    pk[2 * g + 1][x] = sw2[1];
                                }
                                const int chunk = 4 * jj + 2 * g + khalf;  // 8 channels = 16 bytes
                                region[row * 8 + (chunk ^ swz)] = make_uint4(pk[2 * g][0], pk[2 * g][1], pk[2 * g + 1][0], pk[2 * g + 1][1]);
                            }
                        }
                    }
                    uint16_t* obase = reinterpret_cast<uint16_t*>(out) + (int64_t)(m0 + wm * C::WTM + p * 64) * ldo + n0 + wn * C::WTN + jh * 64;
#pragma unroll
                    for (int it = 0; it < 8; it++) {
                        const int q = it * kWave + lane, row = q >> 3, c = q & 7;
                        const uint4 v = region[row * 8 + (c ^ ((row >> 1) & 7))];
                        store_streaming(obase + (int64_t)row * ldo + 8 * c, v);
                    }
                  }
                }
                return;
            }
            float sa_r[C::TM];  // fetched before any store is issued (see above)
#pragma unroll
            for (int i = 0; i < C::TM; i++) sa_r[i] = ep.a_scale ? ep.a_scale[m0 + wm * C::WTM + i * 32 + l32] : 1.f;
#pragma unroll
            for (int j = 0; j < C::TN; j++) {
                const int nb = n0 + wn * C::WTN + j * 32;
                float sw[16], bb[16];
#pragma unroll
                for (int g = 0; g < 4; g++) {
                    const int n = nb + 8 * g + 4 * khalf;
                    if (ep.w_scale) {
                        const float4 v = *reinterpret_cast<const float4*>(ep.w_scale + n);
                        sw[4 * g] = v.x, sw[4 * g + 1] = v.y, sw[4 * g + 2] = v.z, sw[4 * g + 3] = v.w;
                    } else {
                        sw[4 * g] = sw[4 * g + 1] = sw[4 * g + 2] = sw[4 * g + 3] = 1.f;
                    }
#pragma unroll
                    for (int e = 0; e < 4; e++)
                        bb[4 * g + e] = ep.bias ? ep.beta * load_as_f32(ep.bias, ep.bias_dtype, n + e) : 0.f;
                }
#pragma unroll
                for (int i = 0; i < C::TM; i++) {
                    const int m = m0 + wm * C::WTM + i * 32 + l32;
                    const float sa = sa_r[i];
                    uint32_t pk[4][2];
#pragma unroll
                    for (int g = 0; g < 4; g++) {
                        uint16_t h[4];
#pragma unroll
                        for (int e = 0; e < 4; e++) {
                            const auto av = acc[i][j][4 * g + e];
                            h[e] = Lo<ODT>::from_f32(epi_value<PLAIN>((float)av, sa, sw[4 * g + e], alpha, bb[4 * g + e]));
                        }
                        pk[g][0] = (uint32_t)h[0] | ((uint32_t)h[1] << 16);
                        pk[g][1] = (uint32_t)h[2] | ((uint32_t)h[3] << 16);
                    }
                    uint16_t* orow = reinterpret_cast<uint16_t*>(out) + (int64_t)m * ldo;
#pragma unroll
                    for (int g = 0; g < 2; g++) {
#pragma unroll
                        for (int x = 0; x < 2; x++) {
                            const auto sw2 = __builtin_amdgcn_permlane32_swap(pk[2 * g][x], pk[2 * g + 1][x], false, false);
                            pk[2 * g][x] = sw2[0];
                            pk[2 * g + 1][x] = sw2[1];
                        }
                        store_streaming(orow + nb + 16 * g + 8 * khalf, make_uint4(pk[2 * g][0], pk[2 * g][1], pk[2 * g + 1][0], pk[2 * g + 1][1]));
                    }
                }
            }
        };
        if (plain) {
            if (ep.out_dtype == LLMQ_BF16) fast(std::integral_constant<int, LLMQ_BF16>{}, std::true_type{});
            else fast(std::integral_constant<int, LLMQ_F16>{}, std::true_type{});
        } else {
            if (ep.out_dtype == LLMQ_BF16) fast(std::integral_constant<int, LLMQ_BF16>{}, std::false_type{});
            else fast(std::integral_constant<int, LLMQ_F16>{}, std::false_type{});
        }
        return;
    }
#pragma unroll
    for (int j = 0; j < C::TN; j++) {
        const int nb = n0 + wn * C::WTN + j * 32;  // first channel of this 32-wide MFMA tile (wave-uniform)
        if (nb >= N) continue;
        const bool full = nb + 32 <= N;
        float sw[16], bb[16];
#pragma unroll
        for (int r = 0; r < 16; r++) {
            const int n = min(nb + 8 * (r / 4) + 4 * khalf + (r % 4), N - 1);
            sw[r] = (!split && ep.w_scale) ? ep.w_scale[n] : 1.f;
            bb[r] = (!split && ep.bias) ? ep.beta * load_as_f32(ep.bias, ep.bias_dtype, n) : 0.f;
        }
#pragma unroll
        for (int i = 0; i < C::TM; i++) {
            __builtin_amdgcn_sched_barrier(0);  // one tile at a time: keeps the accumulator copies short-lived
            const int m = m0 + wm * C::WTM + i * 32 + l32;
            const bool m_ok = m < M;
            uint32_t raw[16];
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const auto av = acc[i][j][r];  // scalar copy first: bit_cast of a vector element misreads
                raw[r] = __builtin_bit_cast(uint32_t, av);
            }
            if (split || acc_dump) {
                uint32_t* dst = split ? reinterpret_cast<uint32_t*>(partials) + ((int64_t)blockIdx.y * M + m) * N
                                      : reinterpret_cast<uint32_t*>(acc_dump) + (int64_t)m * N;
                if (m_ok) {
#pragma unroll
                    for (int g = 0; g < 4; g++) {
                        const int n = nb + 8 * g + 4 * khalf;
                        if (full && raw_vec) {
                            *reinterpret_cast<uint4*>(dst + n) = make_uint4(raw[4 * g], raw[4 * g + 1], raw[4 * g + 2], raw[4 * g + 3]);
                        } else {
#pragma unroll
                            for (int e = 0; e < 4; e++)
                                if (n + e < N) dst[n + e] = raw[4 * g + e];
                        }
                    }
                }
                if (split) continue;
            }
            const float sa = (ep.a_scale && m_ok) ? ep.a_scale[m] : 1.f;
            uint32_t pk[4][2];  // pk[g] = 4 output elements (channels 8g + 4*khalf .. +3)
#pragma unroll
            for (int g = 0; g < 4; g++) {
                uint16_t h[4];
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    const auto av = acc[i][j][4 * g + e];
                    h[e] = to_out(plain ? epi_value<true>((float)av, sa, sw[4 * g + e], alpha, 0.f) : epi_value<false>((float)av, sa, sw[4 * g + e], alpha, bb[4 * g + e]), ep.out_dtype);
                }
                pk[g][0] = (uint32_t)h[0] | ((uint32_t)h[1] << 16);
                pk[g][1] = (uint32_t)h[2] | ((uint32_t)h[3] << 16);
            }
            if (ep.out_scale) {  // block-uniform: fp32 output, every value through e4m3fn on the stored scale and back
                float* frow = reinterpret_cast<float*>(out) + (int64_t)m * ldo;
                if (m_ok) {
#pragma unroll
                    for (int g = 0; g < 4; g++)
#pragma unroll
                        for (int e = 0; e < 4; e++) {
                            const int n = nb + 8 * g + 4 * khalf + e;
                            const uint16_t h16 = (uint16_t)(pk[g][e >> 1] >> (16 * (e & 1)));
                            const float f = ep.out_dtype == LLMQ_BF16 ? Lo<LLMQ_BF16>::to_f32(h16) : Lo<LLMQ_F16>::to_f32(h16);
                            if (n < N) frow[n] = fp8_round_trip(f, out_scale);
                        }
                }
                continue;
            }
            uint16_t* orow = reinterpret_cast<uint16_t*>(out) + (int64_t)m * ldo;
            if (full && out_vec) {
                // quads 2g and 2g+1 are exchanged between the half-waves: the lower half ends up with
                // channels 16g .. 16g+7 of its token, the upper half with 16g+8 .. 16g+15, so one store
                // instruction writes 32 contiguous bytes per token row
#pragma unroll
                for (int g = 0; g < 2; g++) {
#pragma unroll
                    for (int x = 0; x < 2; x++) {
                        const auto sw2 = __builtin_amdgcn_permlane32_swap(pk[2 * g][x], pk[2 * g + 1][x], false, false);
                        pk[2 * g][x] = sw2[0];
                        pk[2 * g + 1][x] = sw2[1];
                    }
                    if (m_ok)
                        *reinterpret_cast<uint4*>(orow + nb + 16 * g + 8 * khalf) =
                            make_uint4(pk[2 * g][0], pk[2 * g][1], pk[2 * g + 1][0], pk[2 * g + 1][1]);
                }
            } else if (m_ok) {
#pragma unroll
                for (int g = 0; g < 4; g++)
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        const int n = nb + 8 * g + 4 * khalf + e;
                        if (n < N) orow[n] = (uint16_t)(pk[g][e >> 1] >> (16 * (e & 1)));
                    }
            }
        }
    }
}

// Split-K second stage: sum the partial accumulators in split order, then the epilogue.
template <bool FP8>
__global__ __launch_bounds__(256) void splitk_epilogue_kernel(const void* __restrict__ partials, int splits,
                                                              int M, int N, Epilogue ep, void* __restrict__ out,
                                                              int64_t ldo, void* __restrict__ acc_dump) {
    const int64_t total = (int64_t)M * N;
    const float alpha = ep.alpha * (ep.alpha_dev ? *ep.alpha_dev : 1.0f);
    for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
         idx += (int64_t)gridDim.x * blockDim.x) {
        const int m = (int)(idx / N), n = (int)(idx - (int64_t)m * N);
        float accf;
        if (FP8) {
            float s = 0.f;
            for (int i = 0; i < splits; i++) s += reinterpret_cast<const float*>(partials)[i * total + idx];
            if (acc_dump) reinterpret_cast<float*>(acc_dump)[idx] = s;
            accf = s;
        } else {
            int s = 0;
            for (int i = 0; i < splits; i++) s += reinterpret_cast<const int*>(partials)[i * total + idx];
            if (acc_dump) reinterpret_cast<int*>(acc_dump)[idx] = s;
            accf = (float)s;
        }
        const float sa = ep.a_scale ? ep.a_scale[m] : 1.f, sw = ep.w_scale ? ep.w_scale[n] : 1.f;
        const float bb = ep.bias ? ep.beta * load_as_f32(ep.bias, ep.bias_dtype, n) : 0.f;
        const uint16_t h16 = to_out((!ep.bias && alpha == 1.0f) ? epi_value<true>(accf, sa, sw, alpha, 0.f) : epi_value<false>(accf, sa, sw, alpha, bb), ep.out_dtype);
        if (ep.out_scale) {
            const float f = ep.out_dtype == LLMQ_BF16 ? Lo<LLMQ_BF16>::to_f32(h16) : Lo<LLMQ_F16>::to_f32(h16);
            reinterpret_cast<float*>(out)[(int64_t)m * ldo + n] = fp8_round_trip(f, *ep.out_scale);
        } else {
            reinterpret_cast<uint16_t*>(out)[(int64_t)m * ldo + n] = h16;
        }
    }
}

template <class C>
int launch_cfg(const uint8_t* A, int64_t lda, const uint8_t* B, int64_t ldb, int M, int N, int K, const Plan& p,
               const Epilogue& ep, void* out, int64_t ldo, void* acc_dump, void* ws, hipStream_t st) {
    if (C::LDS_BYTES > 65536u) {
        // tiles of more than 64 KB need the limit raised, once per kernel and device
        static bool raised[64] = {};
        int dev = 0;
        if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return LLMQ_ERR_LAUNCH;
        if (!raised[dev]) {
            if (hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_tile_kernel<C, true>),
                                    hipFuncAttributeMaxDynamicSharedMemorySize, (int)C::LDS_BYTES) != hipSuccess)
                return LLMQ_ERR_LAUNCH;
            if constexpr (!C::DMA)
                if (hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_tile_kernel<C, false>),
                                        hipFuncAttributeMaxDynamicSharedMemorySize, (int)C::LDS_BYTES) != hipSuccess)
                    return LLMQ_ERR_LAUNCH;
            raised[dev] = true;  // benign if two threads race here: both set the same value
        }
    }
    const int tiles = cdiv(M, C::BM) * cdiv(N, C::BN);
    // every split covers whole K tiles -> the loads need no K predicate
    const bool kfull = (K % C::BK == 0) && (p.k_per_split % C::BK == 0);
    if constexpr (C::DMA) {
        if (!kfull) return LLMQ_ERR_SHAPE;  // callers route ragged K to the register-staged kernel
        hipLaunchKernelGGL((gemm_tile_kernel<C, true>), dim3(tiles, p.splits), dim3(C::NT), C::LDS_BYTES, st, A, lda, B,
                           ldb, M, N, K, p.k_per_split, ep, out, ldo, acc_dump, ws);
    } else if (kfull)
        hipLaunchKernelGGL((gemm_tile_kernel<C, true>), dim3(tiles, p.splits), dim3(C::NT), C::LDS_BYTES, st, A, lda, B,
                           ldb, M, N, K, p.k_per_split, ep, out, ldo, acc_dump, ws);
    else
        hipLaunchKernelGGL((gemm_tile_kernel<C, false>), dim3(tiles, p.splits), dim3(C::NT), C::LDS_BYTES, st, A, lda,
                           B, ldb, M, N, K, p.k_per_split, ep, out, ldo, acc_dump, ws);
    return launch_status();
}

template <bool FP8, int AFMT, bool DMA>
int launch_shape(const uint8_t* A, int64_t lda, const uint8_t* B, int64_t ldb, int M, int N, int K, const Plan& p,
                 const Epilogue& ep, void* out, int64_t ldo, void* acc_dump, void* ws, hipStream_t st) {
    switch (p.cfg) {
        case 1: return launch_cfg<GemmCfg<256, 256, 64, 2, 4, FP8, AFMT, 2, DMA && !FP8>>(A, lda, B, ldb, M, N, K, p, ep, out, ldo, acc_dump, ws, st);
        case 0: return launch_cfg<GemmCfg<256, 256, 64, 2, 2, FP8, AFMT, 2, DMA && !FP8>>(A, lda, B, ldb, M, N, K, p, ep, out, ldo, acc_dump, ws, st);
        case 2: return launch_cfg<GemmCfg<256, 128, 64, 2, 2, FP8, AFMT, 2, DMA && !FP8>>(A, lda, B, ldb, M, N, K, p, ep, out, ldo, acc_dump, ws, st);
        case 3: return launch_cfg<GemmCfg<128, 128, 64, 2, 2, FP8, AFMT, 2, DMA && !FP8>>(A, lda, B, ldb, M, N, K, p, ep, out, ldo, acc_dump, ws, st);
        case 4: return launch_cfg<GemmCfg<64, 128, 128, 2, 2, FP8, AFMT, 2, DMA>>(A, lda, B, ldb, M, N, K, p, ep, out, ldo, acc_dump, ws, st);
        case 6: return launch_cfg<GemmCfg<256, 256, 128, 2, 4, FP8, AFMT, 1, DMA>>(A, lda, B, ldb, M, N, K, p, ep, out, ldo, acc_dump, ws, st);
        case 7: return launch_cfg<GemmCfg<128, 256, 128, 2, 4, FP8, AFMT, 1, DMA>>(A, lda, B, ldb, M, N, K, p, ep, out, ldo, acc_dump, ws, st);
        default: return launch_cfg<GemmCfg<32, 128, 128, 1, 4, FP8, AFMT, 2, DMA>>(A, lda, B, ldb, M, N, K, p, ep, out, ldo, acc_dump, ws, st);
    }
}

template <bool FP8, int AFMT>
int launch_gemm(const uint8_t* A, int64_t lda, const uint8_t* B, int64_t ldb, int M, int N, int K, const Plan& p,
                const Epilogue& ep, void* out, int64_t ldo, void* acc_dump, void* ws, bool allow_dma, hipStream_t st) {
    // Operand tiles go straight into LDS whenever every split covers whole K tiles (the direct loads cannot zero a
    // ragged tail); llmq_gemm_force_plan(cfg | 64, .) keeps the register-staged loop.  The fp8 K step is 64 bytes, so
    // the 64-byte K tiles have a single sub-step there and stay register-staged.
    const int bk = kShapes[p.cfg].bk;
    const bool dma = allow_dma && K % bk == 0 && p.k_per_split % bk == 0;
    int rc = dma ? launch_shape<FP8, AFMT, true>(A, lda, B, ldb, M, N, K, p, ep, out, ldo, acc_dump, ws, st)
                 : launch_shape<FP8, AFMT, false>(A, lda, B, ldb, M, N, K, p, ep, out, ldo, acc_dump, ws, st);
    if (rc != LLMQ_OK || p.splits == 1) return rc;
    const int64_t total = (int64_t)M * N;
    const int blocks = (int)std::min<int64_t>((total + 255) / 256, 4096);
    hipLaunchKernelGGL((splitk_epilogue_kernel<FP8 || AFMT == 2>), dim3(blocks), dim3(256), 0, st, ws, p.splits, M, N, ep, out, ldo,
                       acc_dump);
    return launch_status();
}

}  // namespace
}  // namespace llmq
