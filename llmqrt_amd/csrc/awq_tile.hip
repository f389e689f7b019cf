// AWQ W4A16 for many tokens: an fp16 MFMA tile GEMM whose weight operand is dequantized on its way
// from global memory into LDS, so that the fp16 weights never exist in HBM
// (the reference dequantizes to HBM and calls a dense matmul above 1024 tokens,
// nn_models/modules/linear/linear_awq.py:47-53; below that its Triton kernel re-reads and
// re-unpacks the weights per 32-token tile, triton_kernels/awq_kernels.py:328-378).
//
// Tile: BM tokens x BN channels x 64 k per step, v_mfma_f32_32x32x16_f16, fp32 accumulators.
//   * activations: fp16 [M, K] rows, 128 bytes per row and K tile, global -> registers -> LDS;
//   * weights: a thread takes the 8 packed words of 8 consecutive k rows at one word column.  That 8x8
//     block of nibbles holds, for each of its 8 channels, exactly the 8 k-consecutive values one MFMA
//     lane operand needs: v_perm_b32 gathers the byte of a nibble pair from two k-adjacent words,
//     (u & 0x000F000F) | 0x64006400 reads as the fp16 pair (1024 + q), a packed add of -(1024 + z) and a
//     packed multiply by the group scale give fp16((q - z) * s) with the reference's single rounding
//     (utils/packing_utils.py:65-80); high nibbles go through (1024 + 16 q) / 16 - (64 + z), also exact.
//     Two threads share a word column (4 channels each); a thread writes four 16-byte LDS chunks per
//     K tile.  Every weight is unpacked once per block, i.e. once per BM tokens.
//   * the weight fragment is the MFMA row operand, so an accumulator quad is 4 consecutive channels of
//     one token and the epilogue stores 16 bytes per lane after one v_permlane32_swap.
// All loads are unconditional with clamped indices (the compiler can then count them); what lies past
// the end of K is zeroed when it is written to LDS, rows past M and channels past N are never stored.
#include <type_traits>

#include "awq_plans.h"
#include "llmq_common.h"

namespace llmq {
namespace {

typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef _Float16 h2 __attribute__((ext_vector_type(2)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef int v4i __attribute__((ext_vector_type(4)));

constexpr int kBK = 64;    // k per tile
constexpr int kCPR = 8;    // 16-byte chunks per LDS row (64 fp16)
constexpr int kNumXcd = 8;
constexpr int kGroupM = 8;

template <int BM_, int BN_, int WM_, int WN_>
struct TileCfg {
    static constexpr int BM = BM_, BN = BN_, WM = WM_, WN = WN_;
    static constexpr int NT = WM * WN * kWave;
    static constexpr int WTM = BM / WM, WTN = BN / WN;
    static constexpr int TM = WTM / 32, TN = WTN / 32;
    static constexpr int A_LOADS = BM * kCPR / NT;
    static constexpr int WORDS = BN / 8;  // word columns of a tile
    static constexpr int STAGE_CHUNKS = (BM + BN) * kCPR;
    static constexpr size_t LDS_BYTES = 2u * STAGE_CHUNKS * 16u;
    static_assert(BM % (WM * 32) == 0 && BN % (WN * 32) == 0, "wave tile must be 32-aligned");
    static_assert((BM * kCPR) % NT == 0, "activation tile must split evenly over threads");
    static_assert(2 * BN == NT, "one weight task (8 k x 4 channels) per thread");
};

// 16-byte chunk c of row `row`; the xor spreads both the row-major activation writes / MFMA operand
// reads (16 consecutive rows, one chunk) and the weight writes (rows 8 apart, one chunk) over the banks.
__device__ __forceinline__ int lds_chunk(int row, int c) { return row * kCPR + (c ^ (((row >> 1) ^ (row >> 3)) & 7)); }

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

// ADMA: the activation tile goes global -> LDS directly (global_load_lds_dwordx4: a lane names its own 16 global
// bytes, a wavefront's 64 pieces land back to back in LDS, so the swizzle is applied on the fetch side); needs whole
// K tiles.  The weights always pass through registers: they are dequantized on the way.
template <class C, bool ADMA>
__global__ __launch_bounds__(C::NT) void awq_tile_kernel(
    const uint16_t* __restrict__ x, int64_t ldx, const uint32_t* __restrict__ qw,
    const uint16_t* __restrict__ scales, const uint32_t* __restrict__ qz, const uint16_t* __restrict__ bias,
    uint16_t* __restrict__ out, float* __restrict__ partials, int M, int N, int K, int G, int k_per_split) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem_raw[];
    uint4* lds = reinterpret_cast<uint4*>(smem_raw);

    const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
    const int wm = wave / C::WN, wn = wave % C::WN;
    const int Nw = N >> 3;
    const int tiles_m = (M + C::BM - 1) / C::BM, tiles_n = (N + C::BN - 1) / C::BN;
    int tile_m, tile_n;
    tile_coords(blockIdx.x, gridDim.x, tiles_m, tiles_n, tile_m, tile_n);
    const int m0 = tile_m * C::BM, n0 = tile_n * C::BN;
    const int k_begin = blockIdx.y * k_per_split;
    const int klen = min(K, k_begin + k_per_split) - k_begin;  // a multiple of 32, at least 32
    const int ktiles = (klen + kBK - 1) / kBK;

    // ---- activations: slot i of a thread is row tid / 8 + i * ROWS_STEP, chunk tid % 8 ------------
    constexpr int ROWS_STEP = C::NT / kCPR;
    const int ld_row = tid / kCPR, ld_c = tid % kCPR;
    const uint16_t* a_base = x + (int64_t)m0 * ldx + k_begin;
    // Row offsets and LDS slots are recomputed per use instead of kept in registers (the 256x256 tile has
    // none to spare); with a row step that is a multiple of 64 the xor term of the slot is the same for all i.
    const int last_row = M - 1 - m0;
    auto a_off = [&](int i) { return min(ld_row + i * ROWS_STEP, last_row) * (int)ldx; };
    const int st_a0 = lds_chunk(ld_row, ld_c);
    auto st_a = [&](int i) {
        return (ROWS_STEP % 64 == 0) ? st_a0 + i * ROWS_STEP * kCPR : lds_chunk(ld_row + i * ROWS_STEP, ld_c);
    };

    // ---- weights: thread = (word column wc, channel half wh, k octet wo) ---------------------------
    const int wc = tid % C::WORDS, wh = (tid / C::WORDS) & 1, wo = tid / (2 * C::WORDS);
    const int cw = min((n0 >> 3) + wc, Nw - 1);  // clamped: channels past N are never stored
    uint32_t magic = 0x64006400u;
    asm volatile("" : "+v"(magic));  // opaque: (u & mask) | magic stays one v_and_or_b32

    uint4 a_reg[ADMA ? 1 : C::A_LOADS];
    uint32_t w_reg[8], z_reg;
    uint4 s_reg;
    const uint32_t lds_base = (uint32_t)(uintptr_t)((__attribute__((address_space(3))) void*)smem_raw);
    const uint32_t wave_off = (uint32_t)__builtin_amdgcn_readfirstlane(wave) * 1024u;
    // direct load of the activation tile kt into `stage`: slot i of a thread lands at chunk (tid + i * NT) of the stage,
    // i.e. row ld_row + i * ROWS_STEP, chunk slot ld_c, which holds global chunk ld_c ^ swizzle(row)
    auto issue_a = [&](int kt, int stage) {
        const int ktc = max(min(kt, ktiles - 1), 0) * kBK;
#pragma unroll
        for (int i = 0; i < C::A_LOADS; i++) {
            const int row = ld_row + i * ROWS_STEP;
            const int gc = ld_c ^ (((row >> 1) ^ (row >> 3)) & 7);
            const uint16_t* src = a_base + a_off(i) + ktc + gc * 8;
            const uint32_t m0v = lds_base + (uint32_t)stage * (C::STAGE_CHUNKS * 16u) + wave_off + (uint32_t)i * (C::NT * 16u);
            asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(m0v), "v"(src) : "memory", "m0");
        }
    };
    auto load_tile = [&](int kt) {
        const int ktc = max(min(kt, ktiles - 1), 0) * kBK;
        if constexpr (!ADMA) {
            const int ka = min(ktc + ld_c * 8, klen - 8);
#pragma unroll
            for (int i = 0; i < C::A_LOADS; i++) a_reg[i] = *reinterpret_cast<const uint4*>(a_base + a_off(i) + ka);
        }
        const int kw = k_begin + min(ktc + wo * 8, klen - 8);
        const uint32_t* wp = qw + (int64_t)kw * Nw + cw;
#pragma unroll
        for (int r = 0; r < 8; r++) w_reg[r] = wp[(int64_t)r * Nw];
        const int g = kw / G;
        z_reg = qz[(int64_t)g * Nw + cw];
        s_reg = *reinterpret_cast<const uint4*>(scales + ((int64_t)g * Nw + cw) * 8);
    };
    auto store_tile = [&](int stage, int kt) {
        uint4* sA = lds + stage * C::STAGE_CHUNKS;
        uint4* sB = sA + C::BM * kCPR;
        if constexpr (!ADMA) {
            const uint32_t keep_a = (kt < ktiles && kt * kBK + ld_c * 8 < klen) ? 0xffffffffu : 0u;
#pragma unroll
            for (int i = 0; i < C::A_LOADS; i++) {
                const uint4 v = a_reg[i];
                sA[st_a(i)] = make_uint4(v.x & keep_a, v.y & keep_a, v.z & keep_a, v.w & keep_a);
            }
        }
        const uint32_t keep_w = (kt < ktiles && kt * kBK + wo * 8 < klen) ? 0xffffffffu : 0u;
        const uint32_t sw[4] = {s_reg.x, s_reg.y, s_reg.z, s_reg.w};
#pragma unroll
        for (int bi = 0; bi < 2; bi++) {
            const uint32_t b = (uint32_t)(2 * wh + bi);  // byte of the word: nibbles 2b (low), 2b + 1 (high)
            const uint32_t sel = b | 0x0c00u | ((4u + b) << 16) | 0x0c000000u;
            uint32_t u[4];
#pragma unroll
            for (int pr = 0; pr < 4; pr++) u[pr] = __builtin_amdgcn_perm(w_reg[2 * pr + 1], w_reg[2 * pr], sel);
#pragma unroll
            for (int hi = 0; hi < 2; hi++) {
                // nibble p = 2b + hi holds channel j = {0,2,4,6,1,3,5,7}[p] = 4 bi + 2 hi + wh of the word
                const uint32_t zq = (z_reg >> (8 * b + 4 * hi)) & 0xFu;
                const uint32_t sh = wh ? (sw[2 * bi + hi] >> 16) : (sw[2 * bi + hi] & 0xffffu);
                const h2 s2 = __builtin_bit_cast(h2, sh * 0x00010001u);
                uint32_t ar[4];
                if (hi) {
                    const h2 cz = __builtin_bit_cast(h2, (0xD400u | (zq << 4)) * 0x00010001u);  // -(64 + z)
                    const h2 k16 = {(_Float16)0.0625f, (_Float16)0.0625f};
#pragma unroll
                    for (int pr = 0; pr < 4; pr++) {
                        const h2 h = __builtin_bit_cast(h2, (u[pr] & 0x00F000F0u) | magic);  // 1024 + 16 q
                        ar[pr] = __builtin_bit_cast(uint32_t, __builtin_elementwise_fma(h, k16, cz) * s2) & keep_w;
                    }
                } else {
                    const h2 cz = __builtin_bit_cast(h2, (0xE400u | zq) * 0x00010001u);  // -(1024 + z)
#pragma unroll
                    for (int pr = 0; pr < 4; pr++) {
                        const h2 h = __builtin_bit_cast(h2, (u[pr] & 0x000F000Fu) | magic);  // 1024 + q
                        ar[pr] = __builtin_bit_cast(uint32_t, (h + cz) * s2) & keep_w;
                    }
                }
                const int nl = 8 * wc + 4 * bi + 2 * hi + wh;  // channel row inside the tile
                sB[lds_chunk(nl, wo)] = make_uint4(ar[0], ar[1], ar[2], ar[3]);
            }
        }
    };
    auto lds_barrier = [] {
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
    };

    v16f acc[C::TM][C::TN];
#pragma unroll
    for (int i = 0; i < C::TM; i++)
#pragma unroll
        for (int j = 0; j < C::TN; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;

    const int l32 = lane & 31, khalf = lane >> 5;
    const int a_row0 = wm * C::WTM + l32, b_row0 = wn * C::WTN + l32;
    auto tile_mfma = [&](int stage) {
        const uint4* sA = lds + stage * C::STAGE_CHUNKS;
        const uint4* sB = sA + C::BM * kCPR;
#pragma unroll
        for (int ks = 0; ks < kBK / 16; ks++) {
            const int c0 = ks * 2 + khalf;
            h8 af[C::TM], bf[C::TN];
#pragma unroll
            for (int i = 0; i < C::TM; i++) af[i] = __builtin_bit_cast(h8, sA[lds_chunk(a_row0 + i * 32, c0)]);
#pragma unroll
            for (int j = 0; j < C::TN; j++) bf[j] = __builtin_bit_cast(h8, sB[lds_chunk(b_row0 + j * 32, c0)]);
#pragma unroll
            for (int i = 0; i < C::TM; i++)
#pragma unroll
                for (int j = 0; j < C::TN; j++)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(bf[j], af[i], acc[i][j], 0, 0, 0);
        }
    };

    // ---- main loop: tile kt is computed from LDS stage kt & 1 while tile kt + 1 waits in registers
    // (dequantized and written to the other stage behind the MFMAs) and tile kt + 2 is in flight ------
    if constexpr (ADMA) {
        // The activation tile kt + 1 is requested at the top of step kt, into the stage that every wavefront finished
        // reading before the last barrier, and has the step's MFMAs to land.  The wait below covers it: it sits before
        // the step's own register loads are issued (a past-the-end tile re-reads the last one into a stage that an
        // all-zero weight tile multiplies, or that nobody reads).
        auto landed = [] { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); };
        issue_a(0, 0);
        load_tile(0);
        store_tile(0, 0);
        landed();
        load_tile(1);
        lds_barrier();
#pragma unroll 1
        for (int kt = 0; kt < ktiles; kt += 2) {
            issue_a(kt + 1, 1);
            tile_mfma(0);
            store_tile(1, kt + 1);
            landed();
            load_tile(kt + 2);
            lds_barrier();
            issue_a(kt + 2, 0);
            tile_mfma(1);  // an odd tile count computes one all-zero tile here
            store_tile(0, kt + 2);
            landed();
            load_tile(kt + 3);
            lds_barrier();
        }
        landed();  // nothing may still be landing in LDS when the block ends
    } else {
        load_tile(0);
        store_tile(0, 0);
        load_tile(1);
        lds_barrier();
#pragma unroll 1
        for (int kt = 0; kt < ktiles; kt += 2) {
            tile_mfma(0);
            store_tile(1, kt + 1);
            load_tile(kt + 2);
            lds_barrier();
            tile_mfma(1);  // an odd tile count computes one all-zero tile here
            store_tile(0, kt + 2);
            load_tile(kt + 3);
            lds_barrier();
        }
    }

    // ---- epilogue: lane = token l32; register r = channel 8 (r / 4) + 4 khalf + r % 4 of the 32-wide tile
    const bool split = gridDim.y > 1;
#pragma unroll
    for (int j = 0; j < C::TN; j++) {
        const int nb = n0 + wn * C::WTN + j * 32;
        if (nb >= N) continue;  // wave-uniform
#pragma unroll
        for (int i = 0; i < C::TM; i++) {
            const int m = m0 + wm * C::WTM + i * 32 + l32;
            const bool m_ok = m < M;
            if (split) {
                float* dst = partials + ((int64_t)blockIdx.y * M + m) * N;
#pragma unroll
                for (int g = 0; g < 4; g++) {
                    const int n = nb + 8 * g + 4 * khalf;
                    if (m_ok && n < N)
                        *reinterpret_cast<float4*>(dst + n) = make_float4(acc[i][j][4 * g], acc[i][j][4 * g + 1],
                                                                          acc[i][j][4 * g + 2], acc[i][j][4 * g + 3]);
                }
                continue;
            }
            uint32_t pk[4][2];
#pragma unroll
            for (int g = 0; g < 4; g++) {
                uint16_t h[4];
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    float v = acc[i][j][4 * g + e];
                    if (bias) {
                        const int n = min(nb + 8 * g + 4 * khalf + e, N - 1);
                        v = Lo<LLMQ_F16>::to_f32(Lo<LLMQ_F16>::from_f32(v)) + Lo<LLMQ_F16>::to_f32(bias[n]);
                    }
                    h[e] = Lo<LLMQ_F16>::from_f32(v);
                }
                pk[g][0] = (uint32_t)h[0] | ((uint32_t)h[1] << 16);
                pk[g][1] = (uint32_t)h[2] | ((uint32_t)h[3] << 16);
            }
            uint16_t* orow = out + (int64_t)m * N;
#pragma unroll
            for (int g = 0; g < 2; g++) {
#pragma unroll
                for (int e = 0; e < 2; e++) {
                    const auto sw2 = __builtin_amdgcn_permlane32_swap(pk[2 * g][e], pk[2 * g + 1][e], false, false);
                    pk[2 * g][e] = sw2[0];
                    pk[2 * g + 1][e] = sw2[1];
                }
                const int n = nb + 16 * g + 8 * khalf;  // 8 consecutive channels; N % 8 == 0: all in or all out
                if (m_ok && n < N)
                    store_streaming(orow + n, make_uint4(pk[2 * g][0], pk[2 * g][1], pk[2 * g + 1][0], pk[2 * g + 1][1]));
            }
        }
    }
}

inline int cdiv(int64_t a, int64_t b) { return (int)((a + b - 1) / b); }

template <class C, bool ADMA>
int launch_tile_impl(const uint16_t* x, int64_t ldx, const uint32_t* qw, const uint16_t* scales, const uint32_t* qz,
                const uint16_t* bias, uint16_t* out, float* ws, int M, int N, int K, int G, int splits, int kps,
                hipStream_t st) {
    auto kernel = awq_tile_kernel<C, ADMA>;
    if (C::LDS_BYTES > 64 * 1024) {
        // per device: the attribute belongs to the loaded code object of the current device
        static bool raised[64] = {};
        int dev = 0;
        if (hipGetDevice(&dev) != hipSuccess) return LLMQ_ERR_LAUNCH;
        if (dev < 0 || dev >= 64 || !raised[dev]) {
            if (hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                    (int)C::LDS_BYTES) != hipSuccess)
                return LLMQ_ERR_LAUNCH;
            if (dev >= 0 && dev < 64) raised[dev] = true;
        }
    }
    const dim3 grid(cdiv(M, C::BM) * cdiv(N, C::BN), splits);
    hipLaunchKernelGGL(kernel, grid, dim3(C::NT), C::LDS_BYTES, st, x, ldx, qw, scales, qz, bias, out, ws, M, N, K, G, kps);
    return launch_status();
}

thread_local int g_awq_tile_dma = 1;  // 0 keeps the register-staged activation loads (tuning / test hook, per host thread)

template <class C>
int launch_tile(const uint16_t* x, int64_t ldx, const uint32_t* qw, const uint16_t* scales, const uint32_t* qz,
                const uint16_t* bias, uint16_t* out, float* ws, int M, int N, int K, int G, int splits, int kps,
                hipStream_t st) {
    // the direct loads cannot zero a ragged K tail; their global addresses must be 16-byte aligned
    const bool dma = g_awq_tile_dma && K % kBK == 0 && kps % kBK == 0 && (ldx & 7) == 0 && (reinterpret_cast<uintptr_t>(x) & 15u) == 0;
    return dma ? launch_tile_impl<C, true>(x, ldx, qw, scales, qz, bias, out, ws, M, N, K, G, splits, kps, st)
               : launch_tile_impl<C, false>(x, ldx, qw, scales, qz, bias, out, ws, M, N, K, G, splits, kps, st);
}

}  // namespace

void set_awq_tile_direct_loads(int on) { g_awq_tile_dma = on; }

AwqTilePlan make_awq_tile_plan(int64_t M, int64_t N, int64_t K, int force_cfg, int force_splits) {
    AwqTilePlan p;
    // Modelled cost = token rows after padding to the tile height x a per-row cost measured on the Qwen2-7B
    // shapes (the larger the tile, the fewer times a weight is dequantized and the fewer LDS bytes per MAC),
    // for the tiles that can fill the GPU: 256x256 needs 400 tiles, 128x128 needs 256 blocks' worth of work
    // (weighted by K, since a long K is split across blocks at little cost).
    const int64_t pad64 = (int64_t)cdiv(M, 64) * 64, pad128 = (int64_t)cdiv(M, 128) * 128, pad256 = (int64_t)cdiv(M, 256) * 256;
    const int64_t tiles256 = (int64_t)cdiv(M, 256) * cdiv(N, 256), blocks128 = (int64_t)cdiv(M, 128) * cdiv(N, 128);
    const double cost64 = (double)pad64;
    const double cost128 = blocks128 * K >= (int64_t)256 * 3584 ? 0.85 * pad128 : 1e30;
    const double cost256 = tiles256 >= 400 ? 0.72 * pad256 : 1e30;
    p.cfg = cost256 <= cost128 && cost256 <= cost64 ? 1 : (cost128 <= cost64 ? 2 : 0);
    if (force_cfg >= 0) p.cfg = force_cfg;
    const int bm = p.cfg == 1 ? 256 : (p.cfg == 2 ? 128 : 64), bn = p.cfg == 1 ? 256 : 128;
    const int blocks = cdiv(M, bm) * cdiv(N, bn);
    const int want = p.cfg == 1 ? 256 : 512;  // blocks that fill the 256 CUs
    int splits = force_splits > 0 ? force_splits : (blocks >= want * 3 / 4 ? 1 : cdiv(want, blocks));
    const int max_splits = (int)(K / 256) > 0 ? (int)(K / 256) : 1;  // at least 4 K tiles per block
    if (splits > max_splits) splits = max_splits;
    if (splits > 32) splits = 32;
    p.k_per_split = cdiv(cdiv(K, splits), kBK) * kBK;
    p.splits = cdiv(K, p.k_per_split);
    return p;
}

int launch_awq_tile(const AwqTilePlan& p, const uint16_t* x, int64_t ldx, const uint32_t* qw, const uint16_t* scales,
                    const uint32_t* qz, const uint16_t* bias, uint16_t* out, float* ws, int M, int N, int K, int G,
                    hipStream_t st) {
    if (p.cfg == 2) return launch_tile<TileCfg<128, 128, 2, 2>>(x, ldx, qw, scales, qz, bias, out, ws, M, N, K, G, p.splits, p.k_per_split, st);
    if (p.cfg == 1) return launch_tile<TileCfg<256, 256, 2, 4>>(x, ldx, qw, scales, qz, bias, out, ws, M, N, K, G, p.splits, p.k_per_split, st);
    return launch_tile<TileCfg<64, 128, 1, 4>>(x, ldx, qw, scales, qz, bias, out, ws, M, N, K, G, p.splits, p.k_per_split, st);
}

}  // namespace llmq
