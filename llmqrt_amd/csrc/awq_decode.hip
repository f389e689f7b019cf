// AWQ W4A16 decode kernel: up to 64 tokens in slabs of 16, group size 128, N a multiple of 32.
//
// The op is a stream of half a byte per weight out of HBM, so the kernel is laid out around the memory
// system first.  Measured on MI355X with a pure-load kernel over the [K, N/8] int32 weight matrix: a
// wavefront load that covers 64-byte row segments streams at 2.5-3.2 TB/s, one that covers whole 128-byte
// lines with 16 bytes per lane at 5.3-5.8 TB/s, provided a few thousand wavefronts each keep about four such
// loads in flight.  Hence:
//   * A block of CS wavefronts owns a column tile of 16*CS packed words (128 or 256 bytes per row) and a run
//     of whole quantization groups along K.  The tile moves in stages of 64 rows: every thread fetches four
//     16-byte pieces (a wavefront instruction covers 4-8 rows x 128-256 contiguous bytes), PD stages ahead of
//     the one being computed, and drops them into a double-buffered LDS tile.
//   * Compute reads LDS in the layout the matrix core wants: wavefront w owns word columns 16w .. 16w+15, a
//     lane the 8 consecutive k-rows of one word column, i.e. an 8x8 block of nibbles = the operand of 8
//     v_mfma_f32_16x16x32_f16 (tokens x 16 channels x 32 k), one per logical column of the word.
//   * Nibbles are not converted: v_perm_b32 puts the same byte of two k-adjacent words into bytes 0 / 2 of a
//     register; masked with 0x000F000F / 0x00F000F0 the nibbles read as fp16 subnormals q * 2^-24 /
//     16 q * 2^-24, which the matrix core multiplies exactly.  Scale and zero point are applied once per
//     group and output: y += s * 2^24 * acc - s * z * sum_k(x), with sum_k(x) from one MFMA against ones.
//     (0.75 VALU operations per weight plus 64 per group and wavefront.)
//   * A K split across blocks writes fp32 partial sums [split][M][N] to the caller's workspace; the block that
//     arrives last at a column tile adds them in split order and writes the output: one launch, results
//     independent of scheduling.  Arrivals are counted in self-resetting tickets at the start of that workspace
//     (cleared once by its owner; calls that may overlap in time use different workspaces).
#include <algorithm>
#include <type_traits>

#include "awq_plans.h"
#include "llmq_common.h"

namespace llmq {

namespace {

typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef int v4i __attribute__((ext_vector_type(4)));
typedef uint32_t u4 __attribute__((ext_vector_type(4)));  // a first-class 16-byte value (HIP's uint4 is a struct: copies of it become memcpy)

constexpr int kGroup = 128;      // quantization group = 2 stages of 64 rows = 4 MFMA chunks of 32 rows
constexpr int kStageRows = 64;

__host__ __device__ constexpr int rev_nibble_d(int j) { return ((j & 1) << 2) | (j >> 1); }  // {0,4,1,5,2,6,3,7}

// Cross-block end of a K split, shared by the decode kernels.  On entry `ptile` (LDS, [M][TILE_CH] fp32) holds this
// block's partial sums for column tile `tile` and every thread of the block has passed a barrier after writing it.
// Every block publishes its tile to partials[ks] (planes of `plane` floats, rows of N); the block that arrives last at the tile adds the splits in
// split order (so the result does not depend on which block that is), adds the bias and writes the output.
// Cross-block visibility without cache-wide fences (a device-scope release fence writes back the whole L2 of the
// XCD: measured at ~100 us per launch): the partial sums are stored and loaded with the device-coherent cache
// policy (sc1: written through / not served from another XCD's stale copy), every wavefront waits until its stores
// have completed before the block takes its ticket, and the ticket is a device-scope atomic.  The coherent stores
// are whole 16-byte pieces of 128-byte lines (4-byte write-through pieces were measured at +11 us per launch).
// Tickets of neighbouring tiles are 256 bytes apart so that their atomics land in different memory channels
// (adjacent words were measured 1-3 us slower per launch).
constexpr int kTicketStride = 64;  // in 4-byte words
template <int TILE_CH, int NT>
__device__ __forceinline__ void finish_split_tile(const float* ptile, int M, int N, int tile, int ks, int splits,
                                                  float* partials, int64_t plane, unsigned int* tickets,
                                                  const uint16_t* bias, uint16_t* out) {
    const int tid = threadIdx.x;
    const int tile_n0 = tile * TILE_CH;                  // first channel of the tile
    const int tile_q = min(TILE_CH, N - tile_n0) >> 2;   // its width in units of 4 channels (N % 32 == 0)
    auto store4 = [&](v4f acc, int m, int nn) __attribute__((always_inline)) {
        float lo0 = acc[0], hi0 = acc[1], lo1 = acc[2], hi1 = acc[3];
        if (bias) {
            lo0 = Lo<LLMQ_F16>::to_f32(Lo<LLMQ_F16>::from_f32(lo0)) + Lo<LLMQ_F16>::to_f32(bias[nn]);
            hi0 = Lo<LLMQ_F16>::to_f32(Lo<LLMQ_F16>::from_f32(hi0)) + Lo<LLMQ_F16>::to_f32(bias[nn + 1]);
            lo1 = Lo<LLMQ_F16>::to_f32(Lo<LLMQ_F16>::from_f32(lo1)) + Lo<LLMQ_F16>::to_f32(bias[nn + 2]);
            hi1 = Lo<LLMQ_F16>::to_f32(Lo<LLMQ_F16>::from_f32(hi1)) + Lo<LLMQ_F16>::to_f32(bias[nn + 3]);
        }
        *reinterpret_cast<uint2*>(out + (int64_t)m * N + nn) =
            make_uint2((uint32_t)Lo<LLMQ_F16>::from_f32(lo0) | ((uint32_t)Lo<LLMQ_F16>::from_f32(hi0) << 16),
                       (uint32_t)Lo<LLMQ_F16>::from_f32(lo1) | ((uint32_t)Lo<LLMQ_F16>::from_f32(hi1) << 16));
    };
    if (splits == 1) {
        for (int idx = tid; idx < M * tile_q; idx += NT) {
            const int m = idx / tile_q, c4 = idx - m * tile_q;
            store4(*reinterpret_cast<const v4f*>(ptile + m * TILE_CH + 4 * c4), m, tile_n0 + 4 * c4);
        }
        return;
    }
    for (int idx = tid; idx < M * tile_q; idx += NT) {
        const int m = idx / tile_q, c4 = idx - m * tile_q;
        const v4f v = *reinterpret_cast<const v4f*>(ptile + m * TILE_CH + 4 * c4);
        float* dst = partials + (int64_t)ks * plane + (int64_t)m * N + tile_n0 + 4 * c4;
        // (the wait states: a 16-byte store reads its data registers after issue, and the compiler does not know that this
        // statement is a store, so it may place a VALU write of those registers right behind it)
        asm volatile("global_store_dwordx4 %0, %1, off sc1\n\ts_nop 1" ::"v"(dst), "v"(v) : "memory");
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // this wavefront's coherent stores have completed
    __shared__ int s_last;
    __syncthreads();
    if (tid == 0) {
        // Arrival ticket of this column tile: counts 0 .. splits-1 and wraps back to 0 with the last arrival, so the
        // slot is clean again for whichever call gets it next.  One atomic per block, no retry loop (a
        // compare-and-swap loop on a shared word was measured at ~1.5 us per arrival, serialized).
        s_last = atomicInc(tickets + kTicketStride * tile, (unsigned)(splits - 1)) == (unsigned)(splits - 1);
    }
    __syncthreads();
    if (!s_last) return;
    // Eight splits at a time, added in split order.  Every coherent load goes to memory, so the read-back costs one round
    // trip per pass: where a pass has more pieces than threads (16 tokens on 512 threads), a thread takes two pieces,
    // sixteen 16-byte loads in flight.
    const int items = M * tile_q;
    auto ld = [&](const float* src, int sp, v4f& t) __attribute__((always_inline)) {
        const float* q = src + (int64_t)min(sp, splits - 1) * plane;
        asm volatile("global_load_dwordx4 %0, %1, off sc1" : "=v"(t) : "v"(q) : "memory");
    };
    auto add8 = [&](v4f& acc, int left, v4f t0, v4f t1, v4f t2, v4f t3, v4f t4, v4f t5, v4f t6, v4f t7) __attribute__((always_inline)) {
        acc += t0;
        if (left > 1) acc += t1;
        if (left > 2) acc += t2;
        if (left > 3) acc += t3;
        if (left > 4) acc += t4;
        if (left > 5) acc += t5;
        if (left > 6) acc += t6;
        if (left > 7) acc += t7;
    };
    for (int base = 0; base < items; base += 2 * NT) {
        const int idx = base + tid, idx1 = idx + NT;
        if (base + NT < items) {  // block-uniform: the second half of the pass is not empty
            const bool two = idx1 < items;  // a lane without a second piece loads its first one twice
            const int ia = idx, ib = two ? idx1 : idx;
            const int ma = ia / tile_q, na = tile_n0 + 4 * (ia - ma * tile_q);
            const int mb = ib / tile_q, nb = tile_n0 + 4 * (ib - mb * tile_q);
            const float* srca = partials + (int64_t)ma * N + na;
            const float* srcb = partials + (int64_t)mb * N + nb;
            v4f acca = {0.f, 0.f, 0.f, 0.f}, accb = {0.f, 0.f, 0.f, 0.f};
            for (int sp = 0; sp < splits; sp += 8) {
                v4f a0, a1, a2, a3, a4, a5, a6, a7, b0, b1, b2, b3, b4, b5, b6, b7;
                ld(srca, sp, a0), ld(srca, sp + 1, a1), ld(srca, sp + 2, a2), ld(srca, sp + 3, a3);
                ld(srca, sp + 4, a4), ld(srca, sp + 5, a5), ld(srca, sp + 6, a6), ld(srca, sp + 7, a7);
                ld(srcb, sp, b0), ld(srcb, sp + 1, b1), ld(srcb, sp + 2, b2), ld(srcb, sp + 3, b3);
                ld(srcb, sp + 4, b4), ld(srcb, sp + 5, b5), ld(srcb, sp + 6, b6), ld(srcb, sp + 7, b7);
                asm volatile("s_waitcnt vmcnt(0)"
                             : "+v"(a0), "+v"(a1), "+v"(a2), "+v"(a3), "+v"(a4), "+v"(a5), "+v"(a6), "+v"(a7), "+v"(b0),
                               "+v"(b1), "+v"(b2), "+v"(b3), "+v"(b4), "+v"(b5), "+v"(b6), "+v"(b7)::"memory");
                add8(acca, splits - sp, a0, a1, a2, a3, a4, a5, a6, a7);
                add8(accb, splits - sp, b0, b1, b2, b3, b4, b5, b6, b7);
            }
            store4(acca, ma, na);
            if (two) store4(accb, mb, nb);
        } else if (idx < items) {
            const int ia = idx;
            const int ma = ia / tile_q, na = tile_n0 + 4 * (ia - ma * tile_q);
            const float* srca = partials + (int64_t)ma * N + na;
            v4f acca = {0.f, 0.f, 0.f, 0.f};
            for (int sp = 0; sp < splits; sp += 8) {
                v4f a0, a1, a2, a3, a4, a5, a6, a7;
                ld(srca, sp, a0), ld(srca, sp + 1, a1), ld(srca, sp + 2, a2), ld(srca, sp + 3, a3);
                ld(srca, sp + 4, a4), ld(srca, sp + 5, a5), ld(srca, sp + 6, a6), ld(srca, sp + 7, a7);
                asm volatile("s_waitcnt vmcnt(0)" : "+v"(a0), "+v"(a1), "+v"(a2), "+v"(a3), "+v"(a4), "+v"(a5), "+v"(a6), "+v"(a7)::"memory");
                add8(acca, splits - sp, a0, a1, a2, a3, a4, a5, a6, a7);
            }
            store4(acca, ma, na);
        }
    }
}

// RM: token rows per lane that can be live (min(M, 4)).  KS: K slices inside the block - KS sets of CS wavefronts, each
// with its own LDS stages, take consecutive shares of the block's groups (KS x the bytes in flight per block at the
// same number of cross-block arrivals) and add their sums through LDS in slice order before the block publishes.
template <int CS, int PD, int RM, int KS>
__global__ __launch_bounds__(CS * KS * kWave, KS == 4 ? 2 : 3) void awq_decode_kernel(
    const uint16_t* __restrict__ x, int64_t ldx, const uint32_t* __restrict__ qw,
    const uint16_t* __restrict__ scales, const uint32_t* __restrict__ qz, const uint16_t* __restrict__ bias,
    uint16_t* __restrict__ out, float* partials, unsigned int* tickets, int Mtot, int N, int K, int gpb, int tiles_n,
    int splits, int slabs) {
    constexpr int NS = CS * kWave, NT = NS * KS;       // threads per slice / per block
    constexpr int SEGW = 16 * CS, SEGQ = SEGW / 4;     // words / 16-byte pieces per tile row
    constexpr int RPL = NS / SEGQ;                     // rows one slice-wide load covers (16)
    constexpr int LOADS = kStageRows / RPL;                          // 16-byte loads per thread and stage (4)
    constexpr int STRIDE = SEGW + 4;  // LDS row stride in words: keeps 16-byte alignment, spreads rows 8 apart over banks
    static_assert(RPL == 16 && LOADS == 4, "a stage is four block-wide loads");
    constexpr int XSTRIDE = 36;       // LDS row stride of the activation tile in words (64 k = 32 words + 4)
    __shared__ __attribute__((aligned(16))) uint32_t lds_all[KS][2][kStageRows * STRIDE];
    __shared__ __attribute__((aligned(16))) uint32_t ldx_all[KS][2][16 * XSTRIDE];  // 16 tokens x 64 k of fp16 per stage

    const int lane = threadIdx.x & (kWave - 1);
    const int wave_b = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    const int slice = wave_b / CS, wave = wave_b % CS;  // wavefront-uniform
    const int tid = threadIdx.x - slice * NS;           // thread index inside the slice
    uint32_t (*lds)[kStageRows * STRIDE] = lds_all[slice];
    uint32_t (*ldx_s)[16 * XSTRIDE] = ldx_all[slice];
    const int li = lane & 15, kb = lane >> 4;
    const int Nw = N >> 3, Nq = Nw >> 2;
    // Work item = (column tile, K split); token slab = 16 tokens.  With several slabs the slabs of a work item sit next
    // to each other on one XCD (flat block ids go round-robin over the 8 XCDs), so the weights cross the fabric once
    // and the other slabs find them in that XCD's L2; blocks past the padded end leave at once.
    int work = blockIdx.x, slab = 0;
    if (slabs > 1) {
        const int q = blockIdx.x >> 3;
        slab = q % slabs;
        work = (q / slabs) * 8 + (blockIdx.x & 7);
        if (work >= tiles_n * splits) return;  // block-uniform, before any barrier
    }
    const int tile = work % tiles_n, ks = work / tiles_n;
    const int M = min(16, Mtot - 16 * slab);  // tokens of this slab
    x += (int64_t)slab * 16 * ldx;
    out += (int64_t)slab * 16 * N;
    if (partials) partials += (int64_t)slab * 16 * N;
    if (tickets) tickets += kTicketStride * tiles_n * slab;
    const int ngroups = K / kGroup;
    const int bg_begin = ks * gpb, bg_end = min(ngroups, bg_begin + gpb);  // the block's groups
    const int per_slice = (bg_end - bg_begin + KS - 1) / KS;
    const int g_first = min(bg_begin + slice * per_slice, bg_end), g_end = min(bg_end, g_first + per_slice);
    const int nst = 2 * (g_end - g_first);          // this slice's stages (0 when the block has fewer groups than slices)
    const int nst_block = 2 * per_slice;            // stages the block steps through (barriers are block-wide)
    const int g_begin = min(g_first, ngroups - 1);  // addressing base: stays inside the matrix for an empty slice
    const int g_last = max(g_end - 1, g_begin);

    // ---- global -> register mapping of the cooperative tile load
    const int ld_row = tid / SEGQ, ld_seg = tid % SEGQ;
    const int colq = min(tile * SEGQ + ld_seg, Nq - 1);  // a tile past the ragged edge re-reads the last piece (unused)
    const u4* wbase = reinterpret_cast<const u4*>(qw) + (int64_t)(g_begin * kGroup + ld_row) * Nq + colq;
    const int st_slot = ld_row * STRIDE + 4 * ld_seg;

    // ---- compute mapping
    const int cw = tile * SEGW + 16 * wave + li;  // word column of this lane
    const bool col_ok = cw < Nw;
    const int cwc = col_ok ? cw : 0;
    // activations: the first 128 threads fetch one 16-byte piece each of the stage's 16 tokens x 64 k
    const bool x_loader = tid < 128;              // wavefront-uniform
    const int x_tok = (tid >> 3) & 15, x_piece = tid & 7;
    const bool x_ok = x_tok < M;
    const uint8_t* xbase = reinterpret_cast<const uint8_t*>(x) +
                           ((int64_t)min(x_tok, M - 1) * ldx + (int64_t)g_begin * kGroup + 8 * x_piece) * 2;
    const int x_slot = x_tok * XSTRIDE + 4 * x_piece;

    struct Stage { u4 w0, w1, w2, w3, x0; };  // one stage in flight: 4 weight pieces, 1 activation piece
    Stage sa, sb;
    uint32_t z_next;
    u4 s_next;
    // every load is unconditional: indices past the block's K range re-read its last stage / group
    auto load_stage = [&](int s, Stage& d) __attribute__((always_inline)) {
        s = min(s, max(nst - 1, 0));
        const u4* p = wbase + (int64_t)s * kStageRows * Nq;
        d.w0 = p[0];
        d.w1 = p[(int64_t)RPL * Nq];
        d.w2 = p[(int64_t)2 * RPL * Nq];
        d.w3 = p[(int64_t)3 * RPL * Nq];
        if (x_loader) d.x0 = *reinterpret_cast<const u4*>(xbase + s * (kStageRows * 2));
    };
    auto load_group = [&](int g) __attribute__((always_inline)) {
        g = min(g, g_last);
        z_next = qz[(int64_t)g * Nw + cwc];
        s_next = *reinterpret_cast<const u4*>(scales + (int64_t)g * N + 8 * cwc);
    };
    auto lds_barrier = []() __attribute__((always_inline)) {  // orders LDS traffic only: the prefetched global loads stay in flight across it
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
    };

    v4f y[8], accg[8], xs = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int j = 0; j < 8; j++) y[j] = accg[j] = v4f{0.f, 0.f, 0.f, 0.f};
    const h8 ones = {(_Float16)1.f, (_Float16)1.f, (_Float16)1.f, (_Float16)1.f,
                     (_Float16)1.f, (_Float16)1.f, (_Float16)1.f, (_Float16)1.f};

    load_group(g_begin);
    load_stage(0, sa);
    if constexpr (PD == 2) load_stage(1, sb);

    uint32_t z_cur = 0;
    u4 s_cur = {0u, 0u, 0u, 0u};

    auto stage_body = [&](int st, Stage& cur) __attribute__((always_inline)) {  // cur: the register set that holds stage st
        const int buf = st & 1;
        uint32_t* tile_lds = lds[buf];
        *reinterpret_cast<u4*>(tile_lds + st_slot) = cur.w0;
        *reinterpret_cast<u4*>(tile_lds + st_slot + RPL * STRIDE) = cur.w1;
        *reinterpret_cast<u4*>(tile_lds + st_slot + 2 * RPL * STRIDE) = cur.w2;
        *reinterpret_cast<u4*>(tile_lds + st_slot + 3 * RPL * STRIDE) = cur.w3;
        if (x_loader) *reinterpret_cast<u4*>(ldx_s[buf] + x_slot) = x_ok ? cur.x0 : u4{0u, 0u, 0u, 0u};  // rows past M read as 0
        if ((st & 1) == 0) {
            z_cur = z_next;
            s_cur = s_next;
            load_group(g_begin + (st >> 1) + 1);
        }
        load_stage(st + PD, cur);
        lds_barrier();
        if (KS > 1 && st >= nst) {  // a slice with fewer stages than the block's longest: barriers only
            __builtin_amdgcn_sched_barrier(0);
            return;
        }
#pragma unroll
        for (int c2 = 0; c2 < 2; c2++) {
            const uint32_t* lp = tile_lds + (32 * c2 + 8 * kb) * STRIDE + 16 * wave + li;
            uint32_t w[8];
#pragma unroll
            for (int r = 0; r < 8; r++) w[r] = lp[r * STRIDE];
            // activation operand: token li, k = 32 c2 + 8 kb .. + 7
            const h8 xb = __builtin_bit_cast(h8, *reinterpret_cast<const u4*>(ldx_s[buf] + li * XSTRIDE + 4 * (4 * c2 + kb)));
            xs = __builtin_amdgcn_mfma_f32_16x16x32_f16(xb, ones, xs, 0, 0, 0);
#pragma unroll
            for (int bsel = 0; bsel < 4; bsel++) {  // byte of the word: nibbles 2*bsel (low) and 2*bsel+1 (high)
                const uint32_t sel = (uint32_t)bsel | 0x0c00u | ((uint32_t)(4 + bsel) << 16) | 0x0c000000u;
                constexpr int kColOfNibble[8] = {0, 2, 4, 6, 1, 3, 5, 7};
                const int jl = kColOfNibble[2 * bsel], jh = kColOfNibble[2 * bsel + 1];
                uint32_t lo[4], hi[4];
#pragma unroll
                for (int pr = 0; pr < 4; pr++) {
                    const uint32_t uu = __builtin_amdgcn_perm(w[2 * pr + 1], w[2 * pr], sel);  // byte0 <- row 2pr, byte2 <- row 2pr+1
                    lo[pr] = uu & 0x000F000Fu;  // q_lo * 2^-24 as fp16 subnormals
                    hi[pr] = uu;                // the whole byte: (16 q_hi + q_lo) * 2^-24, still subnormal and exact
                }
                const h8 bl = __builtin_bit_cast(h8, v4i{(int)lo[0], (int)lo[1], (int)lo[2], (int)lo[3]});
                const h8 bh = __builtin_bit_cast(h8, v4i{(int)hi[0], (int)hi[1], (int)hi[2], (int)hi[3]});
                accg[jl] = __builtin_amdgcn_mfma_f32_16x16x32_f16(xb, bl, accg[jl], 0, 0, 0);
                accg[jh] = __builtin_amdgcn_mfma_f32_16x16x32_f16(xb, bh, accg[jh], 0, 0, 0);
            }
        }
        if (st & 1) {
            // Finished group.  Per byte of the word the accumulators hold L = sum x q_lo 2^-24 (low-nibble column jl)
            // and U = sum x (16 q_hi + q_lo) 2^-24 (high-nibble column jh), so
            //   y_jl += s_jl 2^24 L - s_jl z_jl sum(x),   y_jh += s_jh 2^20 (U - L) - s_jh z_jh sum(x);
            // the group accumulators restart at 0.  Rows past RM belong to tokens past M: their operand rows are zero.
            const uint32_t sw[4] = {s_cur[0], s_cur[1], s_cur[2], s_cur[3]};
            auto scale_of = [&](int j) __attribute__((always_inline)) {
                return Lo<LLMQ_F16>::to_f32((uint16_t)((j & 1) ? (sw[j >> 1] >> 16) : (sw[j >> 1] & 0xffffu)));
            };
#pragma unroll
            for (int bsel = 0; bsel < 4; bsel++) {
                constexpr int kColOfNibble[8] = {0, 2, 4, 6, 1, 3, 5, 7};
                const int jl = kColOfNibble[2 * bsel], jh = kColOfNibble[2 * bsel + 1];
                const float sl = scale_of(jl), sh = scale_of(jh);
                const float zl = (float)((z_cur >> (8 * bsel)) & 0xFu), zh = (float)((z_cur >> (8 * bsel + 4)) & 0xFu);
                const float sl24 = sl * 16777216.0f, sh20 = sh * 1048576.0f, nslz = -sl * zl, nshz = -sh * zh;
#pragma unroll
                for (int r = 0; r < RM; r++) {
                    const float L = accg[jl][r], U = accg[jh][r];
                    y[jl][r] = fmaf(sl24, L, fmaf(nslz, xs[r], y[jl][r]));
                    y[jh][r] = fmaf(sh20, U, fmaf(-sh20, L, fmaf(nshz, xs[r], y[jh][r])));
                    accg[jl][r] = 0.f;
                    accg[jh][r] = 0.f;
                }
            }
            xs = v4f{0.f, 0.f, 0.f, 0.f};
        }
        // Nothing of the next stage may move above this point: its LDS stores wait for its global loads, which
        // were issued at the top of this stage and need this stage's compute time to arrive.
        __builtin_amdgcn_sched_barrier(0);
    };

    // stages alternate between the PD register sets; nst is even, PD is 1 or 2
#pragma unroll 1
    for (int st = 0; st < nst_block; st += 2) {
        stage_body(st, sa);
        if constexpr (PD == 2) stage_body(st + 1, sb);
        else stage_body(st + 1, sa);
    }

    // ---- store: lane (word column li, quarter kb) holds tokens 4*kb + r for its 8 channels
    const int n = 8 * cw;
    auto finish8 = [&](const float* v, int m, int nn) __attribute__((always_inline)) {  // 8 channels -> fp16 (+ bias), one 16-byte store
        uint32_t o[4];
#pragma unroll
        for (int j = 0; j < 4; j++) {
            float lo = v[2 * j], hi = v[2 * j + 1];
            if (bias) {
                lo = Lo<LLMQ_F16>::to_f32(Lo<LLMQ_F16>::from_f32(lo)) + Lo<LLMQ_F16>::to_f32(bias[nn + 2 * j]);
                hi = Lo<LLMQ_F16>::to_f32(Lo<LLMQ_F16>::from_f32(hi)) + Lo<LLMQ_F16>::to_f32(bias[nn + 2 * j + 1]);
            }
            o[j] = (uint32_t)Lo<LLMQ_F16>::from_f32(lo) | ((uint32_t)Lo<LLMQ_F16>::from_f32(hi) << 16);
        }
        *reinterpret_cast<uint4*>(out + (int64_t)m * N + nn) = make_uint4(o[0], o[1], o[2], o[3]);
    };
    if (KS == 1 && splits == 1) {
        if (!col_ok) return;
#pragma unroll
        for (int r = 0; r < RM; r++) {
            const int m = 4 * kb + r;
            if (m >= M) continue;
            const float v[8] = {y[0][r], y[1][r], y[2][r], y[3][r], y[4][r], y[5][r], y[6][r], y[7][r]};
            finish8(v, m, n);
        }
        return;
    }
    constexpr int TILE_CH = SEGW * 8;  // channels per tile
    float* ptile = reinterpret_cast<float*>(&lds_all[0][0][0]);  // [M][TILE_CH] fp32, reuses the weight stages
    static_assert(2 * kStageRows * STRIDE >= 16 * TILE_CH, "the partial tile fits in the weight stages");
    __syncthreads();  // every wavefront is done reading the last stage
#pragma unroll
    for (int sl = 0; sl < KS; sl++) {  // slice 0 writes its sums, the others add theirs in slice order
        if (sl == slice) {
#pragma unroll
            for (int r = 0; r < RM; r++) {
                const int m = 4 * kb + r;
                if (m >= M) continue;
                float4* dst = reinterpret_cast<float4*>(ptile + m * TILE_CH + (16 * wave + li) * 8);
                float4 a = make_float4(y[0][r], y[1][r], y[2][r], y[3][r]), b = make_float4(y[4][r], y[5][r], y[6][r], y[7][r]);
                if (sl > 0) {
                    const float4 pa = dst[0], pb = dst[1];
                    a = make_float4(pa.x + a.x, pa.y + a.y, pa.z + a.z, pa.w + a.w);
                    b = make_float4(pb.x + b.x, pb.y + b.y, pb.z + b.z, pb.w + b.w);
                }
                dst[0] = a;
                dst[1] = b;
            }
        }
        __syncthreads();
    }
    finish_split_tile<TILE_CH, NT>(ptile, M, N, tile, ks, splits, partials, (int64_t)Mtot * N, tickets, bias, out);
}

inline int cdiv_d(int64_t a, int64_t b) { return (int)((a + b - 1) / b); }

}  // namespace

bool awq_decode_supported(int64_t M, int64_t N, int64_t K, int64_t group) {
    // a call's tickets (one per column tile and token slab) must fit in the ticket area of the workspace
    return M >= 1 && M <= 64 && group == kGroup && (N % 32) == 0 && (K % kGroup) == 0 &&
           (size_t)((M + 15) / 16) * (N / 256 + 1) * kTicketStride * sizeof(unsigned int) <= kAwqTicketBytes;
}

// Column tile width (CS wavefronts = 16*CS words), prefetch depth, K slices per block and K split.  Measured on the
// Qwen2-7B shapes (weights streamed from HBM): 128-byte row segments (CS = 2) with one stage in flight beat the wider
// tile and the deeper prefetch everywhere.  About 2048 wavefronts fill the chip, but a column tile should see at most
// ~40 arrivals (its ticket is one memory word: arrivals serialize at ~50 ns each), and the fp32 partial sums, written
// through and read back coherently by the one block that finishes a tile, grow with splits x tokens: the more tokens,
// the fewer blocks along K and the more K slices inside a block (bytes in flight without more arrivals).
//   wide N (column tiles alone nearly fill the chip; gate_up): one slice and blocks of 6 groups up to 6 tokens
//     (16.2 / 17.9 us at 1 / 4 tokens; blocks of 4 groups, i.e. 7 splits, measured 17.9 / 20.7 on the same box: the
//     partial sums and arrivals of the extra splits cost more than their wavefronts bring), 2 slices x 5 groups at
//     7-8 (19.7), beyond that 4 slices and no split across blocks (22.1 at 16 tokens; the register-streaming kernel
//     needs 24.1);
//   long K (down): 4 slices of ~3 groups (12.0 us at one token against 13.9 with one slice; 17.3 at 16);
//   short K, narrow N (qkv, o): 2 slices of one group up to 4 tokens (6.7 us at one token against 7.5; 8.4 at 4
//     against 10.8), 4 slices of one group beyond (8.9 at 8, 10.7 at 16 tokens);
//   17-64 tokens run as slabs of 16 tokens that share the weights through one XCD's L2: qkv 12.3 us at 32 and 14.4
//     at 64 tokens (register-streaming kernel + finish kernel: 13.8 / 19.8), o 11.7 / 13.5 (13.1 / 17.5), gate_up
//     33.2 / 43.8 (39.2 / 57.1), down 21.1 / 28.8 (22.4 / 31.1).
AwqDecodePlan make_awq_decode_plan(int64_t M, int64_t N, int64_t K, int force_cs, int force_pd, int force_splits, int force_ks) {
    const int groups = (int)(K / kGroup), Nw = (int)(N / 8);
    AwqDecodePlan p;
    p.cs = force_cs > 0 ? force_cs : 2;
    p.pd = force_pd > 0 ? force_pd : 1;
    const int strips = cdiv_d(Nw, 16);  // wavefront-wide column strips
    int s = cdiv_d(2048, strips);       // enough wavefronts
    if (s > 40) s = 40;
    if (M > 16) {
        // Token slabs multiply the blocks: keep them all resident at once (4 slices = 92 KB of LDS, one block per CU;
        // 2 slices = 46 KB, three) - a second round of blocks costs more than any split gains.
        const int slabs = cdiv_d(M, 16), tiles = cdiv_d(strips, 2) * slabs;
        p.ks = tiles <= 256 ? 4 : 2;
        const int fit = std::max(1, (p.ks == 4 ? 256 : 768) / tiles);
        if (strips >= 128) s = p.ks == 4 ? 1 : std::min(fit, 2);
        else if (K >= 8192) s = std::min(cdiv_d(groups, 11), fit);
        else s = std::min(cdiv_d(groups, 4), fit);
    } else if (strips >= 128) {
        if (M <= 6) p.ks = 1, s = std::min(s, cdiv_d(groups, 6));
        else if (M <= 8) p.ks = 2, s = std::min(s, cdiv_d(groups, 10));
        else p.ks = 4, s = 1;
    } else if (K >= 8192) {
        p.ks = 4, s = std::min(s, cdiv_d(groups, 11));
    } else if (M <= 4) {
        p.ks = 2, s = (int)std::min<int64_t>(std::min(s, groups / 2), std::max<int64_t>(groups / M, 1));
    } else {
        p.ks = 4, s = std::min(s, cdiv_d(groups, 4));
    }
    if (force_ks == 1 || force_ks == 2 || force_ks == 4) p.ks = force_ks;
    if (p.cs != 2 || p.pd != 1) p.ks = 1;  // the slices exist for the 128-byte tile with one stage ahead only
    if (force_splits > 0) s = force_splits;
    if (s > groups) s = groups;
    if (s < 1) s = 1;
    p.groups_per_block = cdiv_d(groups, s);
    if (force_splits <= 0) p.groups_per_block = cdiv_d(p.groups_per_block, p.ks) * p.ks;  // equal shares for the slices
    p.splits = cdiv_d(groups, p.groups_per_block);
    return p;
}

// fp32 partial sums [splits][M][N]
size_t awq_decode_workspace_bytes(const AwqDecodePlan& p, int64_t M, int64_t N) {
    return p.splits > 1 ? (size_t)p.splits * M * N * sizeof(float) : 0;
}

// Arrival tickets: one counter per column tile and token slab, kTicketStride words apart, at the start of the caller's
// workspace (kAwqTicketBytes).  They must be zero when a call starts and are zero again when it ends (each returns to
// zero with its last arrival), so a workspace is cleared once, when it is allocated, and calls that may overlap in
// time use different workspaces, exactly as for the partial sums behind them.  The library keeps no state of its own.
__global__ void awq_clear_tickets_kernel(unsigned int* p, size_t n) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) p[i] = 0u;
}

int awq_clear_tickets(void* workspace, size_t bytes, hipStream_t st) {
    const size_t n = (bytes < kAwqTicketBytes ? bytes : kAwqTicketBytes) / sizeof(unsigned int);
    if (n == 0) return LLMQ_OK;
    hipLaunchKernelGGL(awq_clear_tickets_kernel, dim3(64), dim3(256), 0, st, static_cast<unsigned int*>(workspace), n);
    return launch_status();
}

int launch_awq_decode(const AwqDecodePlan& p, const uint16_t* x, int64_t ldx, const uint32_t* qw, const uint16_t* scales,
                      const uint32_t* qz, const uint16_t* bias, uint16_t* out, unsigned int* tickets, float* ws, int M,
                      int N, int K, hipStream_t st) {
    const int tiles_n = cdiv_d(N / 8, 16 * p.cs);
    const int slabs = cdiv_d(M, 16), work = tiles_n * p.splits;
    const dim3 grid((unsigned)(slabs == 1 ? work : cdiv_d(work, 8) * 8 * slabs));
    if (p.splits > 1 && (!tickets || (size_t)tiles_n * slabs * kTicketStride * sizeof(unsigned int) > kAwqTicketBytes))
        return LLMQ_ERR_WORKSPACE;
#define LLMQ_DECODE_RM(CS_, PD_, RM_, KS_)                                                                            \
    hipLaunchKernelGGL((awq_decode_kernel<CS_, PD_, RM_, KS_>), grid, dim3(CS_ * KS_ * kWave), 0, st, x, ldx, qw, scales, \
                       qz, bias, out, ws, tickets, M, N, K, p.groups_per_block, tiles_n, p.splits, slabs)
#define LLMQ_DECODE(CS_, PD_, KS_)                         \
    do {                                                   \
        if (M == 1) LLMQ_DECODE_RM(CS_, PD_, 1, KS_);      \
        else if (M == 2) LLMQ_DECODE_RM(CS_, PD_, 2, KS_); \
        else LLMQ_DECODE_RM(CS_, PD_, 4, KS_);             \
    } while (0)
    if (p.cs == 4 && p.pd == 2) LLMQ_DECODE(4, 2, 1);
    else if (p.cs == 4) LLMQ_DECODE(4, 1, 1);
    else if (p.pd == 2) LLMQ_DECODE(2, 2, 1);
    else if (p.ks == 4) LLMQ_DECODE(2, 1, 4);
    else if (p.ks == 2) LLMQ_DECODE(2, 1, 2);
    else LLMQ_DECODE(2, 1, 1);
#undef LLMQ_DECODE
#undef LLMQ_DECODE_RM
    return launch_status();
}

}  // namespace llmq
