// AWQ W4A16: group-dequant GEMM for decode shapes and the standalone dequantizer.
//
// Weight layout (nn_models/modules/linear/linear_awq.py:192-202): qweight int32 [K, N/8];
// nibble p of a word holds logical column 8c + {0,2,4,6,1,3,5,7}[p], i.e. logical column j is
// nibble REV[j] with REV = {0,4,1,5,2,6,3,7} (utils/packing_utils.py:5).  qzeros [K/G, N/8]
// uses the same packing, scales are fp16 [K/G, N].
//
// GEMM kernel.  The op is HBM-bound (half a byte per weight), so the only goal is to stream
// qweight at full rate and keep the unpack cheap enough for the VALU to keep up:
//   * out^T = W^T x^T on v_mfma_f32_16x16x32_f16: the MFMA "A" rows are 16 output channels,
//     the "B" columns are up to 16 tokens, both operands want 8 consecutive k per lane.
//   * A lane loads the words of 8 consecutive k-rows for its word column(s) with plain
//     coalesced global loads (no LDS): that 8x8 block of nibbles is the A operand of 8 MFMAs,
//     one per logical column j.  For column j, v_perm_b32 pulls the byte that holds nibble
//     REV[j] out of two k-adjacent words into the low bytes of the two halves of a register;
//     (u & 0x000F000F) | 0x64006400 then reads as two fp16 values 1024+q (low nibble) or
//     (u & 0x00F000F0) | 0x64006400 as 1024+16q (high nibble); one packed add / fma removes
//     the bias and the zero point exactly, one packed multiply applies the group scale with
//     the same single fp16 rounding as the reference dequantizer.  ~2 VALU ops per weight.
//   * fp32 accumulation in the MFMA; the 4 wavefronts of a block split the block's K range and
//     are summed through LDS in a fixed order; a K split across blocks goes through an fp32
//     workspace and a finishing kernel, again in a fixed order (results are deterministic).
#include "awq_plans.h"
#include "llmq_common.h"

namespace llmq {


namespace {

typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef _Float16 h2 __attribute__((ext_vector_type(2)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef int v4i __attribute__((ext_vector_type(4)));

__host__ __device__ constexpr int rev_nibble(int j) { return ((j & 1) << 2) | (j >> 1); }  // {0,4,1,5,2,6,3,7}

template <int V> struct WordVec;
template <> struct WordVec<1> { typedef uint32_t type; };
template <> struct WordVec<2> { typedef uint2 type; };
template <> struct WordVec<4> { typedef uint4 type; };

template <int V> __device__ __forceinline__ uint32_t word_of(const typename WordVec<V>::type& v, int t);
template <> __device__ __forceinline__ uint32_t word_of<1>(const uint32_t& v, int) { return v; }
template <> __device__ __forceinline__ uint32_t word_of<2>(const uint2& v, int t) { return t ? v.y : v.x; }
template <> __device__ __forceinline__ uint32_t word_of<4>(const uint4& v, int t) {
    return t == 0 ? v.x : (t == 1 ? v.y : (t == 2 ? v.z : v.w));
}

constexpr int kChunkK = 32;  // k per MFMA step
constexpr int kBlockWaves = 4;

// V: words (of 8 columns) per lane -> a wavefront covers 128*V output channels.
// MT: 16-token tiles (M <= 16*MT).
template <int V, int MT>
__global__ __launch_bounds__(kBlockWaves * kWave) void awq_gemm_kernel(
    const uint16_t* __restrict__ x, int64_t ldx, const uint32_t* __restrict__ qw,
    const uint16_t* __restrict__ scales, const uint32_t* __restrict__ qz, const uint16_t* __restrict__ bias,
    uint16_t* __restrict__ out, float* __restrict__ partials, int M, int N, int K, int G, int chunks_per_block) {
    typedef typename WordVec<V>::type wvec;
    constexpr int NACC = MT * V * 8;
    __shared__ float4 red[NACC * kWave];

    const int lane = threadIdx.x & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);  // wave-uniform: keeps the K-range branches scalar
    const int li = lane & 15, kb = lane >> 4;
    const int Nw = N >> 3;
    const int cw = blockIdx.x * (16 * V) + V * li;  // first word column of this lane
    const bool col_ok = cw < Nw;
    const int cwc = col_ok ? cw : 0;

    const int total_chunks = K / kChunkK;
    const int cb0 = blockIdx.y * chunks_per_block, cb1 = min(total_chunks, cb0 + chunks_per_block);
    const int cpw = (cb1 - cb0 + kBlockWaves - 1) / kBlockWaves;
    const int c0 = cb0 + wave * cpw, c1 = min(cb1, c0 + cpw);

    v4f acc[MT][V][8];
#pragma unroll
    for (int a = 0; a < MT; a++)
#pragma unroll
        for (int t = 0; t < V; t++)
#pragma unroll
            for (int j = 0; j < 8; j++) acc[a][t][j] = v4f{0.f, 0.f, 0.f, 0.f};

    h2 cz[V][8], s2[V][8];  // per-group constants: -(bias+zero) and the scale, both halves equal
    int cur_g = -1;

    // Chunk ring: 4 chunks of packed words (+ their activations) are in flight per wavefront, so a
    // chunk's loads are issued three chunk-times before they are consumed; the zeros / scales of the
    // next group are fetched while the current group is being processed.
    constexpr int RING = 4;
    wvec wr[RING][8];
    uint4 xr[RING][MT];
    auto load_chunk = [&](int c, wvec* wdst, uint4* xdst) {
        const int k0 = c * kChunkK + 8 * kb;
        const uint32_t* wp = qw + (int64_t)k0 * Nw + cwc;
#pragma unroll
        for (int r = 0; r < 8; r++) wdst[r] = *reinterpret_cast<const wvec*>(wp + (int64_t)r * Nw);
#pragma unroll
        for (int a = 0; a < MT; a++) {
            const int m = a * 16 + li;
            xdst[a] = m < M ? *reinterpret_cast<const uint4*>(x + (int64_t)m * ldx + k0) : make_uint4(0, 0, 0, 0);
        }
    };
    wvec zv_next;
    uint4 sv_next[V];
    auto load_group = [&](int g) {
        zv_next = *reinterpret_cast<const wvec*>(qz + (int64_t)g * Nw + cwc);
#pragma unroll
        for (int t = 0; t < V; t++)
            sv_next[t] = *reinterpret_cast<const uint4*>(scales + (int64_t)g * N + 8 * (cwc + t));
    };
    // 0x64006400 kept in a register the optimizer cannot see through, so that (u & mask) | magic is one
    // v_and_or_b32 (a VOP3 instruction may carry only one literal)
    uint32_t magic = 0x64006400u;
    asm volatile("" : "+v"(magic));

    const int ngroups = K / G;
    if (c0 < c1) load_group((c0 * kChunkK) / G);
#pragma unroll
    for (int u = 0; u < RING; u++)
        if (c0 + u < c1) load_chunk(c0 + u, wr[u], xr[u]);

    auto process = [&](int c, const wvec* wcur, const uint4* xcur) {
        const int g = (c * kChunkK) / G;
        if (g != cur_g) {
            cur_g = g;
            const wvec zv = zv_next;
            uint4 sv[V];
#pragma unroll
            for (int t = 0; t < V; t++) sv[t] = sv_next[t];
            if (g + 1 < ngroups && ((g + 1) * G) / kChunkK < c1) load_group(g + 1);
#pragma unroll
            for (int t = 0; t < V; t++) {
                const uint32_t zw = word_of<V>(zv, t);
                const uint32_t sw[4] = {sv[t].x, sv[t].y, sv[t].z, sv[t].w};
#pragma unroll
                for (int j = 0; j < 8; j++) {
                    constexpr uint32_t kLoBase = 0xE400u, kHiBase = 0xD400u;  // -(1024), -(64) as fp16 bits
                    const int p = rev_nibble(j);
                    const uint32_t z = (zw >> (4 * p)) & 0xFu;
                    const uint32_t c16 = (p & 1) ? (kHiBase | (z << 4)) : (kLoBase | z);  // -(64+z) / -(1024+z)
                    cz[t][j] = __builtin_bit_cast(h2, c16 * 0x00010001u);
                    const uint32_t sh = (j & 1) ? (sw[j >> 1] >> 16) : (sw[j >> 1] & 0xffffu);
                    s2[t][j] = __builtin_bit_cast(h2, sh * 0x00010001u);
                }
            }
        }
        h8 xb[MT];
#pragma unroll
        for (int a = 0; a < MT; a++) xb[a] = __builtin_bit_cast(h8, xcur[a]);
#pragma unroll
        for (int t = 0; t < V; t++) {
#pragma unroll
            for (int j = 0; j < 8; j++) {
                const int p = rev_nibble(j);
                const uint32_t sel = (uint32_t)(p >> 1) | 0x0c00u | ((uint32_t)(4 + (p >> 1)) << 16) | 0x0c000000u;
                uint32_t ar[4];
#pragma unroll
                for (int pr = 0; pr < 4; pr++) {
                    const uint32_t w0 = word_of<V>(wcur[2 * pr], t), w1 = word_of<V>(wcur[2 * pr + 1], t);
                    const uint32_t u = __builtin_amdgcn_perm(w1, w0, sel);  // byte0 <- w0, byte2 <- w1
                    h2 d;
                    if (p & 1) {
                        const h2 h = __builtin_bit_cast(h2, (u & 0x00F000F0u) | magic);  // 1024 + 16 q
                        const h2 k16 = {(_Float16)0.0625f, (_Float16)0.0625f};
                        d = __builtin_elementwise_fma(h, k16, cz[t][j]);                 // q - z, exact
                    } else {
                        const h2 h = __builtin_bit_cast(h2, (u & 0x000F000Fu) | magic);  // 1024 + q
                        d = h + cz[t][j];                                                // q - z, exact
                    }
                    ar[pr] = __builtin_bit_cast(uint32_t, d * s2[t][j]);  // fp16((q - z) * s), one rounding
                }
                const h8 af = __builtin_bit_cast(h8, v4i{(int)ar[0], (int)ar[1], (int)ar[2], (int)ar[3]});
#pragma unroll
                for (int a = 0; a < MT; a++)
                    acc[a][t][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(af, xb[a], acc[a][t][j], 0, 0, 0);
            }
        }
    };

    for (int c = c0; c < c1; c += RING) {
#pragma unroll
        for (int u = 0; u < RING; u++) {
            if (c + u < c1) {
                process(c + u, wr[u], xr[u]);
                if (c + u + RING < c1) load_chunk(c + u + RING, wr[u], xr[u]);
            }
        }
    }

    // ---- sum the 4 wavefronts in wave order through LDS ---------------------------------------
    for (int src = 1; src < kBlockWaves; src++) {
        __syncthreads();
        if (wave == src) {
#pragma unroll
            for (int a = 0; a < MT; a++)
#pragma unroll
                for (int t = 0; t < V; t++)
#pragma unroll
                    for (int j = 0; j < 8; j++) {
                        const v4f v = acc[a][t][j];
                        red[((a * V + t) * 8 + j) * kWave + lane] = make_float4(v[0], v[1], v[2], v[3]);
                    }
        }
        __syncthreads();
        if (wave == 0) {
#pragma unroll
            for (int a = 0; a < MT; a++)
#pragma unroll
                for (int t = 0; t < V; t++)
#pragma unroll
                    for (int j = 0; j < 8; j++) {
                        const float4 v = red[((a * V + t) * 8 + j) * kWave + lane];
                        acc[a][t][j] += v4f{v.x, v.y, v.z, v.w};
                    }
        }
    }
    if (wave != 0) return;

    // ---- store: lane (token li, quarter kb) holds rows 4*kb + r of every MFMA tile, i.e. the 8
    // consecutive channels 8*(cw_tile + V*(4*kb + r) + t) + j, j = 0..7 ------------------------
    const bool split = gridDim.y > 1;
#pragma unroll
    for (int a = 0; a < MT; a++) {
        const int m = a * 16 + li;
        if (m >= M) continue;
#pragma unroll
        for (int t = 0; t < V; t++) {
#pragma unroll
            for (int r = 0; r < 4; r++) {
                const int wcol = blockIdx.x * (16 * V) + V * (4 * kb + r) + t;
                if (wcol >= Nw) continue;
                const int n = 8 * wcol;
                float v[8];
#pragma unroll
                for (int j = 0; j < 8; j++) v[j] = acc[a][t][j][r];
                if (split) {
                    float4* dst = reinterpret_cast<float4*>(partials + ((int64_t)blockIdx.y * M + m) * N + n);
                    dst[0] = make_float4(v[0], v[1], v[2], v[3]);
                    dst[1] = make_float4(v[4], v[5], v[6], v[7]);
                } else {
                    uint32_t o[4];
#pragma unroll
                    for (int j = 0; j < 4; j++) {
                        float lo = v[2 * j], hi = v[2 * j + 1];
                        if (bias) {
                            lo = Lo<LLMQ_F16>::to_f32(Lo<LLMQ_F16>::from_f32(lo)) + Lo<LLMQ_F16>::to_f32(bias[n + 2 * j]);
                            hi = Lo<LLMQ_F16>::to_f32(Lo<LLMQ_F16>::from_f32(hi)) + Lo<LLMQ_F16>::to_f32(bias[n + 2 * j + 1]);
                        }
                        o[j] = (uint32_t)Lo<LLMQ_F16>::from_f32(lo) | ((uint32_t)Lo<LLMQ_F16>::from_f32(hi) << 16);
                    }
                    *reinterpret_cast<uint4*>(out + (int64_t)m * N + n) = make_uint4(o[0], o[1], o[2], o[3]);
                }
            }
        }
    }
}

// Decode kernel (16 tokens per block, up to 4 such slabs per launch; group size 128).  Same streaming scheme, with the scale and the zero point
// moved out of the per-weight work.  The raw nibbles go to the matrix core as fp16 SUBNORMALS:
// (u & 0x000F000F) read as two fp16 values is q * 2^-24 (a high nibble, u & 0x00F000F0, is
// 16 q * 2^-24); their products with fp16 activations are exact in the fp32 accumulator.  Per
// quantization group and output channel
//   y[m,n] += s[n] * 2^24 * acc[m,n]  -  s[n] * z[n] * xsum[m],
// where xsum[m] = sum_k x[m,k] over the group comes from one extra MFMA against a vector of ones.
// Unpacking is one v_perm_b32 per two k-pairs plus one v_and_b32 per pair (0.75 VALU op per weight),
// and two FMAs per group and output.  The tokens are the MFMA rows and the lane's own word columns the
// MFMA columns, so each lane needs exactly the zeros word and the 8 scales of the columns it streams.
// Weights are never rounded to fp16 here (the reference dequantizer rounds (q - z) * s once): the
// result is the exact-weight product, well inside the tolerance of that math.
//
// Work unit = one group = 4 chunks of 32 k.  The loop body is branch-free: every load is issued
// unconditionally (indices clamped to the wavefront's last group) so that the compiler can count the
// loads in flight and wait only for the oldest ring slot; 4 chunks (+ the next group's zeros/scales)
// stay in flight per wavefront.
template <int V, int KW, int MS>
__global__ __launch_bounds__(KW * kWave) void awq_gemv_kernel(
    const uint16_t* __restrict__ x, int64_t ldx, const uint32_t* __restrict__ qw,
    const uint16_t* __restrict__ scales, const uint32_t* __restrict__ qz, const uint16_t* __restrict__ bias,
    uint16_t* __restrict__ out, float* __restrict__ partials, int M_total, int N, int K, int slabs) {
    typedef typename WordVec<V>::type wvec;
    constexpr int G = 128, RING = G / kChunkK, NACC = MS * V * 8;
    constexpr int TOK = 16 * MS;  // tokens per block: MS MFMA token tiles share every unpacked weight operand
    // With several token tiles the per-group rescaling of the accumulators (two fused multiply-adds per
    // accumulator element and group, plus the moves between the two register files) outweighs what the
    // subnormal operands save in unpacking: those variants dequantize each weight to fp16((q - z) * s), as
    // the reference dequantizer rounds it, and accumulate straight into y.
    constexpr bool EX = MS > 1;
    __shared__ float4 red[(KW / 2) * NACC * kWave];

    const int lane = threadIdx.x & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);  // scalar: keeps the loop bounds uniform
    const int li = lane & 15, kb = lane >> 4;
    const int Nw = N >> 3;
    // Column tile and token slab of this block.  Consecutive block ids are dealt round-robin to the 8
    // XCDs; give each XCD a contiguous range of (tile, slab) pairs instead, so that the two 64-byte halves
    // of a cache line (adjacent tiles when V == 1) and the up to 4 token slabs of 16 rows that stream the
    // same weights are served by the same L2 at about the same time (HBM sees the weights once).
    int seq = blockIdx.x;
    {
        const int nb = gridDim.x, q = nb / 8, r = nb % 8, xcd = seq % 8, local = seq / 8;
        seq = xcd < r ? xcd * (q + 1) + local : r * (q + 1) + (xcd - r) * q + local;
    }
    const int tile = seq / slabs, slab = seq - tile * slabs;
    const int M = min(TOK, M_total - TOK * slab);  // tokens of this slab
    x += (int64_t)(TOK * slab) * ldx;
    out += (int64_t)(TOK * slab) * N;
    partials += (int64_t)(TOK * slab) * N;
    const int cw = tile * (16 * V) + V * li;  // first word column of this lane
    const bool col_ok = cw < Nw;
    const int cwc = col_ok ? cw : 0;

    // Groups are dealt cyclically over all gridDim.y * KW wavefronts that share a column tile: at any
    // moment they work on neighbouring groups, so the whole grid sweeps one compact window of rows
    // down the matrix (DRAM pages are used up while open) instead of gridDim.y * KW distant ones.
    const int ngroups = K / G;
    const int gstride = (int)gridDim.y * KW;
    const int g0 = (int)blockIdx.y * KW + wave;

    v4f y[MS][V][8], accg[MS][V][8], xs[MS];
#pragma unroll
    for (int a = 0; a < MS; a++) {
        xs[a] = v4f{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int t = 0; t < V; t++)
#pragma unroll
            for (int j = 0; j < 8; j++) {
                y[a][t][j] = v4f{0.f, 0.f, 0.f, 0.f};
                accg[a][t][j] = v4f{0.f, 0.f, 0.f, 0.f};
            }
    }

    if (g0 < ngroups) {
        wvec wr[RING][8];
        uint4 xr[RING][MS];
        uint32_t voff[8];  // loop-invariant row offsets; the chunk base is wave-uniform
#pragma unroll
        for (int r = 0; r < 8; r++) voff[r] = (uint32_t)(((8 * kb + r) * Nw + cwc) * 4);
        uint32_t xoff[MS];
#pragma unroll
        for (int a = 0; a < MS; a++) xoff[a] = (uint32_t)((min(16 * a + li, M - 1) * (int)ldx + 8 * kb) * 2);
        // loads past the last group of this wavefront re-read that group (results unused): no branches
        auto load_chunk = [&](int g, int u, wvec* wdst, uint4* xdst) {
            const int c = (g < ngroups ? g : g - gstride) * RING + u;
            const uint8_t* wbase = reinterpret_cast<const uint8_t*>(qw) + (int64_t)c * kChunkK * Nw * 4;
#pragma unroll
            for (int r = 0; r < 8; r++) wdst[r] = *reinterpret_cast<const wvec*>(wbase + voff[r]);
#pragma unroll
            for (int a = 0; a < MS; a++)
                xdst[a] = *reinterpret_cast<const uint4*>(reinterpret_cast<const uint8_t*>(x) + (int64_t)c * kChunkK * 2 + xoff[a]);
        };
        wvec z_cur, z_next;
        uint4 s_cur[V], s_next[V];
        auto load_group = [&](int g) {
            g = g < ngroups ? g : g - gstride;
            z_next = *reinterpret_cast<const wvec*>(qz + (int64_t)g * Nw + cwc);
#pragma unroll
            for (int t = 0; t < V; t++)
                s_next[t] = *reinterpret_cast<const uint4*>(scales + (int64_t)g * N + 8 * (cwc + t));
        };
        const h8 ones = {(_Float16)1.f, (_Float16)1.f, (_Float16)1.f, (_Float16)1.f,
                         (_Float16)1.f, (_Float16)1.f, (_Float16)1.f, (_Float16)1.f};
        uint32_t magic = 0x64006400u;
        asm volatile("" : "+v"(magic));  // opaque: (u & mask) | magic stays one v_and_or_b32
        bool row_ok[MS];
#pragma unroll
        for (int a = 0; a < MS; a++) row_ok[a] = 16 * a + li < M;

        // same issue order as in the loop (group, slot 0..3), pinned, so that the wait counts the compiler
        // derives at the loop head are those of the steady state
        load_group(g0);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int u = 0; u < RING; u++) {
            load_chunk(g0, u, wr[u], xr[u]);
            __builtin_amdgcn_sched_barrier(0);
        }

#pragma unroll 1
        for (int g = g0; g < ngroups; g += gstride) {
            z_cur = z_next;
#pragma unroll
            for (int t = 0; t < V; t++) s_cur[t] = s_next[t];
            load_group(g + gstride);
            h2 cz[V][8], s2[V][8];  // EX: -(1024 + z) or -(64 + z), and the scale, both halves equal
            if constexpr (EX) {
#pragma unroll
                for (int t = 0; t < V; t++) {
                    const uint32_t zw = word_of<V>(z_cur, t);
                    const uint32_t sw[4] = {s_cur[t].x, s_cur[t].y, s_cur[t].z, s_cur[t].w};
#pragma unroll
                    for (int j = 0; j < 8; j++) {
                        const int p = rev_nibble(j);
                        const uint32_t z = (zw >> (4 * p)) & 0xFu;
                        const uint32_t c16 = (p & 1) ? (0xD400u | (z << 4)) : (0xE400u | z);
                        cz[t][j] = __builtin_bit_cast(h2, c16 * 0x00010001u);
                        const uint32_t sh = (j & 1) ? (sw[j >> 1] >> 16) : (sw[j >> 1] & 0xffffu);
                        s2[t][j] = __builtin_bit_cast(h2, sh * 0x00010001u);
                    }
                }
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int u = 0; u < RING; u++) {
                h8 xb[MS];
#pragma unroll
                for (int a = 0; a < MS; a++) {
                    uint4 xv = xr[u][a];
                    if (!row_ok[a]) xv = make_uint4(0, 0, 0, 0);
                    xb[a] = __builtin_bit_cast(h8, xv);
                    if constexpr (!EX) xs[a] = __builtin_amdgcn_mfma_f32_16x16x32_f16(xb[a], ones, xs[a], 0, 0, 0);
                }
#pragma unroll
                for (int t = 0; t < V; t++) {
#pragma unroll
                    for (int bsel = 0; bsel < 4; bsel++) {  // byte of the word: nibbles 2*bsel (low), 2*bsel+1 (high)
                        const uint32_t sel = (uint32_t)bsel | 0x0c00u | ((uint32_t)(4 + bsel) << 16) | 0x0c000000u;
                        constexpr int kColOfNibble[8] = {0, 2, 4, 6, 1, 3, 5, 7};  // logical column of nibble p
                        const int jl = kColOfNibble[2 * bsel], jh = kColOfNibble[2 * bsel + 1];
                        uint32_t lo[4], hi[4];
#pragma unroll
                        for (int pr = 0; pr < 4; pr++) {
                            const uint32_t w0 = word_of<V>(wr[u][2 * pr], t), w1 = word_of<V>(wr[u][2 * pr + 1], t);
                            const uint32_t uu = __builtin_amdgcn_perm(w1, w0, sel);  // byte0 <- w0, byte2 <- w1
                            if constexpr (EX) {
                                const h2 hl = __builtin_bit_cast(h2, (uu & 0x000F000Fu) | magic);  // 1024 + q
                                const h2 hh = __builtin_bit_cast(h2, (uu & 0x00F000F0u) | magic);  // 1024 + 16 q
                                const h2 k16 = {(_Float16)0.0625f, (_Float16)0.0625f};
                                lo[pr] = __builtin_bit_cast(uint32_t, (hl + cz[t][jl]) * s2[t][jl]);
                                hi[pr] = __builtin_bit_cast(uint32_t, __builtin_elementwise_fma(hh, k16, cz[t][jh]) * s2[t][jh]);
                            } else {
                                lo[pr] = uu & 0x000F000Fu;  // q * 2^-24 as fp16 subnormals
                                hi[pr] = uu & 0x00F000F0u;  // 16 q * 2^-24
                            }
                        }
                        const h8 bl = __builtin_bit_cast(h8, v4i{(int)lo[0], (int)lo[1], (int)lo[2], (int)lo[3]});
                        const h8 bh = __builtin_bit_cast(h8, v4i{(int)hi[0], (int)hi[1], (int)hi[2], (int)hi[3]});
#pragma unroll
                        for (int a = 0; a < MS; a++) {
                            if constexpr (EX) {
                                y[a][t][jl] = __builtin_amdgcn_mfma_f32_16x16x32_f16(xb[a], bl, y[a][t][jl], 0, 0, 0);
                                y[a][t][jh] = __builtin_amdgcn_mfma_f32_16x16x32_f16(xb[a], bh, y[a][t][jh], 0, 0, 0);
                            } else {
                                accg[a][t][jl] = __builtin_amdgcn_mfma_f32_16x16x32_f16(xb[a], bl, accg[a][t][jl], 0, 0, 0);
                                accg[a][t][jh] = __builtin_amdgcn_mfma_f32_16x16x32_f16(xb[a], bh, accg[a][t][jh], 0, 0, 0);
                            }
                        }
                    }
                }
                // keep the issue order: this slot's refill goes out only now, and nothing of the next
                // chunk is scheduled above it (the waits then cover only the oldest slot)
                __builtin_amdgcn_sched_barrier(0);
                load_chunk(g + gstride, u, wr[u], xr[u]);
                __builtin_amdgcn_sched_barrier(0);
            }
            // y += s * 2^24 * acc - s * z * xsum for this group; the group accumulators restart at 0
            if constexpr (!EX) {
#pragma unroll
            for (int t = 0; t < V; t++) {
                const uint32_t zw = word_of<V>(z_cur, t);
                const uint32_t sw[4] = {s_cur[t].x, s_cur[t].y, s_cur[t].z, s_cur[t].w};
#pragma unroll
                for (int j = 0; j < 8; j++) {
                    const int p = rev_nibble(j);
                    const float zf = (float)((zw >> (4 * p)) & 0xFu);
                    const float sf = Lo<LLMQ_F16>::to_f32((uint16_t)((j & 1) ? (sw[j >> 1] >> 16) : (sw[j >> 1] & 0xffffu)));
                    const float s1 = sf * ((p & 1) ? 1048576.0f : 16777216.0f);  // 2^20 for 16 q, 2^24 for q
                    const float sz = -sf * zf;
#pragma unroll
                    for (int a = 0; a < MS; a++)
#pragma unroll
                        for (int r = 0; r < 4; r++) {
                            y[a][t][j][r] = fmaf(s1, accg[a][t][j][r], fmaf(sz, xs[a][r], y[a][t][j][r]));
                            accg[a][t][j][r] = 0.f;
                        }
                }
            }
#pragma unroll
            for (int a = 0; a < MS; a++) xs[a] = v4f{0.f, 0.f, 0.f, 0.f};
            }
        }
    }

    // ---- sum the KW wavefronts through LDS: a fixed binary tree (upper half adds into lower half) -----
#pragma unroll
    for (int half = KW / 2; half >= 1; half /= 2) {
        __syncthreads();
        if (wave >= half && wave < 2 * half) {
#pragma unroll
            for (int a = 0; a < MS; a++)
#pragma unroll
                for (int t = 0; t < V; t++)
#pragma unroll
                    for (int j = 0; j < 8; j++) {
                        const v4f v = y[a][t][j];
                        red[((wave - half) * NACC + (a * V + t) * 8 + j) * kWave + lane] = make_float4(v[0], v[1], v[2], v[3]);
                    }
        }
        __syncthreads();
        if (wave < half) {
#pragma unroll
            for (int a = 0; a < MS; a++)
#pragma unroll
                for (int t = 0; t < V; t++)
#pragma unroll
                    for (int j = 0; j < 8; j++) {
                        const float4 v = red[(wave * NACC + (a * V + t) * 8 + j) * kWave + lane];
                        y[a][t][j] += v4f{v.x, v.y, v.z, v.w};
                    }
        }
    }
    if (wave != 0 || !col_ok) return;

    // ---- store: lane (word column li, quarter kb) holds tokens 16*a + 4*kb + r for its 8*V channels ---
    const bool split = gridDim.y > 1;
#pragma unroll
    for (int a = 0; a < MS; a++) {
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const int m = 16 * a + 4 * kb + r;
            if (m >= M) continue;
#pragma unroll
            for (int t = 0; t < V; t++) {
                const int n = 8 * (cw + t);
                if (split) {
                    float4* dst = reinterpret_cast<float4*>(partials + ((int64_t)blockIdx.y * M_total + m) * N + n);
                    dst[0] = make_float4(y[a][t][0][r], y[a][t][1][r], y[a][t][2][r], y[a][t][3][r]);
                    dst[1] = make_float4(y[a][t][4][r], y[a][t][5][r], y[a][t][6][r], y[a][t][7][r]);
                } else {
                    uint32_t o[4];
#pragma unroll
                    for (int j = 0; j < 4; j++) {
                        float lo = y[a][t][2 * j][r], hi = y[a][t][2 * j + 1][r];
                        if (bias) {
                            lo = Lo<LLMQ_F16>::to_f32(Lo<LLMQ_F16>::from_f32(lo)) + Lo<LLMQ_F16>::to_f32(bias[n + 2 * j]);
                            hi = Lo<LLMQ_F16>::to_f32(Lo<LLMQ_F16>::from_f32(hi)) + Lo<LLMQ_F16>::to_f32(bias[n + 2 * j + 1]);
                        }
                        o[j] = (uint32_t)Lo<LLMQ_F16>::from_f32(lo) | ((uint32_t)Lo<LLMQ_F16>::from_f32(hi) << 16);
                    }
                    *reinterpret_cast<uint4*>(out + (int64_t)m * N + n) = make_uint4(o[0], o[1], o[2], o[3]);
                }
            }
        }
    }
}

// Cross-block split-K finish: sum partials in split order, round to fp16, add bias.
__global__ __launch_bounds__(256) void awq_finish_kernel(const float* __restrict__ partials, int splits, int64_t total,
                                                         int N, const uint16_t* __restrict__ bias,
                                                         uint16_t* __restrict__ out) {
    for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
         idx += (int64_t)gridDim.x * blockDim.x) {
        float s = 0.f;
        for (int i = 0; i < splits; i++) s += partials[i * total + idx];
        if (bias) s = Lo<LLMQ_F16>::to_f32(Lo<LLMQ_F16>::from_f32(s)) + Lo<LLMQ_F16>::to_f32(bias[idx % N]);
        out[idx] = Lo<LLMQ_F16>::from_f32(s);
    }
}

// Standalone dequantizer: one thread per packed word -> 8 fp16 (16-byte store).
__global__ __launch_bounds__(256) void awq_dequant_kernel(const uint32_t* __restrict__ qw,
                                                          const uint16_t* __restrict__ scales,
                                                          const uint32_t* __restrict__ qz, uint16_t* __restrict__ out,
                                                          int64_t K, int Nw, int G) {
    const int64_t total = K * Nw;
    for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
         idx += (int64_t)gridDim.x * blockDim.x) {
        const int64_t k = idx / Nw;
        const int c = (int)(idx - k * Nw);
        const int64_t g = k / G;
        const uint32_t w = qw[idx], z = qz[g * Nw + c];
        const uint4 sv = *reinterpret_cast<const uint4*>(scales + (g * Nw + c) * 8);
        const uint32_t sw[4] = {sv.x, sv.y, sv.z, sv.w};
        uint32_t o[4];
#pragma unroll
        for (int j2 = 0; j2 < 4; j2++) {
            uint32_t pair = 0;
#pragma unroll
            for (int h = 0; h < 2; h++) {
                const int j = 2 * j2 + h, sh = 4 * rev_nibble(j);
                const int d = (int)((w >> sh) & 0xFu) - (int)((z >> sh) & 0xFu);
                const _Float16 s = __builtin_bit_cast(_Float16, (uint16_t)(h ? (sw[j2] >> 16) : (sw[j2] & 0xffffu)));
                const _Float16 v = (_Float16)d * s;  // exact difference, one fp16 RNE multiply
                pair |= (uint32_t)__builtin_bit_cast(uint16_t, v) << (16 * h);
            }
            o[j2] = pair;
        }
        *reinterpret_cast<uint4*>(out + idx * 8) = make_uint4(o[0], o[1], o[2], o[3]);
    }
}

// Dequantizer for group sizes that are multiples of 8 (all real checkpoints): a wavefront owns 64 word
// columns x 8 consecutive K rows, which lie in one group, so zeros and scales are loaded once per 8 words
// and all 8 word loads are in flight together.  Nibbles p and p + 4 of a word are adjacent columns, so one
// shift + mask yields two columns as the fp16 pair (1024 + q_lo, 1024 + q_hi); subtracting (1024 + z) is
// exact and the packed fp16 multiply by the scale pair rounds once, like the scalar kernel above.
__global__ __launch_bounds__(256) void awq_dequant_rows_kernel(const uint32_t* __restrict__ qw,
                                                               const uint16_t* __restrict__ scales,
                                                               const uint32_t* __restrict__ qz,
                                                               uint16_t* __restrict__ out, int K, int Nw, int G) {
    constexpr int R = 8;
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    const int c = blockIdx.x * kWave + lane;
    const int k0 = ((int)blockIdx.y * 4 + wave) * R;
    if (c >= Nw || k0 >= K) return;
    const int64_t g = k0 / G;
    uint32_t w[R];
#pragma unroll
    for (int r = 0; r < R; r++) w[r] = qw[(int64_t)(k0 + r) * Nw + c];
    const uint32_t z = qz[g * Nw + c];
    const uint4 sv = *reinterpret_cast<const uint4*>(scales + (g * Nw + c) * 8);
    const uint32_t sw[4] = {sv.x, sv.y, sv.z, sv.w};
    h2 zp[4], sp[4];
#pragma unroll
    for (int j = 0; j < 4; j++) {
        zp[j] = __builtin_bit_cast(h2, ((z >> (4 * j)) & 0x000F000Fu) | 0x64006400u);
        sp[j] = __builtin_bit_cast(h2, sw[j]);
    }
#pragma unroll
    for (int r = 0; r < R; r++) {
        uint32_t o[4];
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const h2 q = __builtin_bit_cast(h2, ((w[r] >> (4 * j)) & 0x000F000Fu) | 0x64006400u);
            o[j] = __builtin_bit_cast(uint32_t, (q - zp[j]) * sp[j]);
        }
        *reinterpret_cast<uint4*>(out + ((int64_t)(k0 + r) * Nw + c) * 8) = make_uint4(o[0], o[1], o[2], o[3]);
    }
}

// Dequantizer that writes the transpose, fp16 [N, K] with K contiguous: the operand layout of the MFMA GEMM
// (llmq_gemm_f16), for the many-token path.  Same arithmetic as awq_dequant_rows_kernel (bit-identical values).  A
// thread owns 8 consecutive K rows of one word column, i.e. 8 k-values of 8 channels = one 16-byte piece of 8 output
// rows; the lanes of a wavefront are (k octet, word column) = (lane % 8, lane / 8), so that a store instruction writes
// 8 channel rows x 128 contiguous bytes, and the 4 wavefronts of a block read the four 32-byte quarters of the same
// packed 128-byte line.
__global__ __launch_bounds__(256) void awq_dequant_t_kernel(const uint32_t* __restrict__ qw,
                                                             const uint16_t* __restrict__ scales,
                                                             const uint32_t* __restrict__ qz,
                                                             uint16_t* __restrict__ out, int K, int Nw, int G) {
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    const int c = blockIdx.x * 32 + wave * 8 + (lane >> 3);
    const int k0 = (int)blockIdx.y * 64 + (lane & 7) * 8;
    if (c >= Nw || k0 >= K) return;
    const int64_t g = k0 / G;
    uint32_t w[8];
#pragma unroll
    for (int r = 0; r < 8; r++) w[r] = qw[(int64_t)(k0 + r) * Nw + c];
    const uint32_t z = qz[g * Nw + c];
    const uint4 sv = *reinterpret_cast<const uint4*>(scales + (g * Nw + c) * 8);
    const uint32_t sw[4] = {sv.x, sv.y, sv.z, sv.w};
    uint32_t o[8][4];  // o[r][j]: channels 2j (low half) and 2j + 1 (high half) of row k0 + r
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const h2 zp = __builtin_bit_cast(h2, ((z >> (4 * j)) & 0x000F000Fu) | 0x64006400u);
        const h2 sp = __builtin_bit_cast(h2, sw[j]);
#pragma unroll
        for (int r = 0; r < 8; r++) {
            const h2 q = __builtin_bit_cast(h2, ((w[r] >> (4 * j)) & 0x000F000Fu) | 0x64006400u);
            o[r][j] = __builtin_bit_cast(uint32_t, (q - zp) * sp);
        }
    }
#pragma unroll
    for (int j = 0; j < 4; j++) {
#pragma unroll
        for (int h = 0; h < 2; h++) {
            const uint32_t sel = h ? 0x07060302u : 0x05040100u;  // the high / low halves of two registers
            uint32_t v[4];
#pragma unroll
            for (int pr = 0; pr < 4; pr++) v[pr] = __builtin_amdgcn_perm(o[2 * pr + 1][j], o[2 * pr][j], sel);
            *reinterpret_cast<uint4*>(out + (int64_t)(8 * c + 2 * j + h) * K + k0) = make_uint4(v[0], v[1], v[2], v[3]);
        }
    }
}

struct AwqPlan { int v, mt, splits, chunks_per_block; };

inline int cdiv(int64_t a, int64_t b) { return (int)((a + b - 1) / b); }

thread_local int g_force_v = 0, g_force_splits = 0, g_force_kw = 0;  // tuning hook (llmq_awq_force_plan): per host thread

// Generic kernel (any group size, up to 64 tokens): 4 wavefronts split the block's K range.
AwqPlan make_awq_plan(int64_t M, int64_t N, int64_t K) {
    AwqPlan p;
    p.mt = cdiv(M, 16);
    const int Nw = (int)(N / 8);
    p.v = 1;
    if (g_force_v == 2 && p.mt == 1 && Nw % 2 == 0) p.v = 2;
    const int ntiles = cdiv(Nw, 16 * p.v);
    const int chunks = (int)(K / kChunkK);
    // aim at ~2 blocks per CU; every wavefront should keep at least 4 chunks
    int splits = g_force_splits > 0 ? g_force_splits : cdiv(512, ntiles);
    const int max_splits = chunks / (4 * kBlockWaves) > 0 ? chunks / (4 * kBlockWaves) : 1;
    if (splits > max_splits) splits = max_splits;
    if (splits < 1) splits = 1;
    p.chunks_per_block = cdiv(cdiv(chunks, splits), 4) * 4;
    p.splits = cdiv(chunks, p.chunks_per_block);
    return p;
}

// Decode kernel (group 128): a block = one column tile x one 16-token slab x KW wavefronts along K; a K split
// across blocks only when the tiles alone cannot fill the GPU.
struct DecodePlan { int v, kw, ms, splits; };
DecodePlan make_decode_plan(int64_t M, int64_t N, int64_t K) {
    DecodePlan p;
    const int Nw = (int)(N / 8), groups = (int)(K / 128);
    // Token tiles of 16 per wavefront.  Above 16 tokens, for a long K that is split across blocks anyway
    // (down), one wavefront feeds every unpacked weight operand to 2 or 4 token tiles instead of running
    // one block per 16-token slab: measured at 64 tokens with the weights coming from HBM, down 30.5 -> 27 us.
    // For K = 3584 the slabs are as fast or faster (qkv 19 vs 21.6 us, gate_up 57 vs 65 us).
    p.ms = (cdiv(Nw, 16) < 128 && K >= 8192) ? (M > 32 ? 4 : (M > 16 ? 2 : 1)) : 1;
    if (g_force_v == 5) p.ms = 2;
    if (g_force_v == 6) p.ms = 4;
    if (g_force_v == 1 || g_force_v == 2) p.ms = 1;
    // 128-byte row segments (V = 2) stream measurably faster than 64-byte ones; use them whenever
    // the tiles alone give every other CU a block, and then do without a second kernel.  With more than one
    // 16-token slab per column tile the narrower tiles are slightly ahead: twice the blocks, two per CU
    // instead of one (gate_up at 64 tokens: 58 -> 56.6 us from HBM, 52 -> 43 us with cache-resident weights).
    p.v = (p.ms == 1 && M <= 16 && Nw % 2 == 0 && Nw / 32 >= 128) ? 2 : 1;
    if (p.ms == 1 && (g_force_v == 1 || (g_force_v == 2 && Nw % 2 == 0))) p.v = g_force_v;
    p.kw = ((g_force_kw == 4 || g_force_kw == 8) && p.v == 1 && p.ms == 1) ? g_force_kw : 4;
    const int ntiles = cdiv(Nw, 16 * p.v);
    int splits = g_force_splits > 0 ? g_force_splits : (ntiles >= 128 ? 1 : cdiv(200, ntiles));  // measured optimum: ~200 blocks
    if (splits > groups / p.kw) splits = groups / p.kw;  // at least one group per wavefront
    if (splits < 1) splits = 1;
    p.splits = splits;
    return p;
}

// The streaming kernel handles up to 64 tokens per weight pass as up to 4 slabs of 16.
inline bool decode_path(int64_t M, int64_t group) { return M <= 64 && group == 128; }

// The LDS-staged decode kernel (one launch, in-kernel K-split reduction) serves up to 64 tokens (slabs of 16) wherever
// its shape conditions hold (group 128, N a multiple of 32); with the K slices and splits of make_awq_decode_plan it
// is level with or ahead of the register-streaming kernel on every measured shape (o at 16 tokens 10.4 against 10.1 us
// is the one tie; at 64 tokens qkv 14.4 against 19.8, gate_up 43.8 against 57.1, down 28.8 against 31.1).
// llmq_awq_force_plan 8..11 picks its tile width and prefetch depth, 1 / 2 / 5 / 6 keep the register-streaming kernel.
inline bool decode16_path(int64_t M, int64_t N, int64_t K, int64_t group) {
    return ((g_force_v == 0 && M <= 64) || (g_force_v >= 8 && g_force_v <= 11)) && awq_decode_supported(M, N, K, group);
}
inline AwqDecodePlan decode16_plan(int64_t M, int64_t N, int64_t K) {
    const int cs = g_force_v >= 8 ? ((g_force_v & 1) ? 4 : 2) : 0, pd = g_force_v >= 8 ? (g_force_v >= 10 ? 2 : 1) : 0;
    return make_awq_decode_plan(M, N, K, cs, pd, g_force_splits, g_force_kw);
}

// More than 64 tokens go to the tile kernel (weights dequantized once per token tile on their way into LDS);
// llmq_awq_force_plan(3 | 4, ...) forces its 64x128 | 256x256 tile for any M, (1 | 2, ...) keeps the slabs.
inline bool tile_path(int64_t M) { return g_force_v == 3 || g_force_v == 4 || g_force_v == 7 || (g_force_v == 0 && M > 64); }
inline AwqTilePlan tile_plan(int64_t M, int64_t N, int64_t K) {
    return make_awq_tile_plan(M, N, K, (g_force_v == 3 || g_force_v == 4) ? g_force_v - 3 : (g_force_v == 7 ? 2 : -1), g_force_splits);
}

template <int V, int MT>
void launch_awq(const AwqPlan& p, const uint16_t* x, int64_t ldx, const uint32_t* qw, const uint16_t* scales,
                const uint32_t* qz, const uint16_t* bias, uint16_t* out, float* ws, int M, int N, int K, int G,
                hipStream_t st) {
    const int ntiles = cdiv(N / 8, 16 * V);
    hipLaunchKernelGGL((awq_gemm_kernel<V, MT>), dim3(ntiles, p.splits), dim3(kBlockWaves * kWave), 0, st, x, ldx, qw,
                       scales, qz, bias, out, ws, M, N, K, G, p.chunks_per_block);
}

}  // namespace
}  // namespace llmq

using namespace llmq;

extern "C" int llmq_awq_force_plan(int v, int splits, int k_waves) {
    const int staged = v >= 0 ? (v & 32) : 0;  // + 32: the tile kernel keeps its register-staged activation loads
    if (v >= 0) v &= ~32;
    if (v < 0 || v > 11 || splits < 0 || splits > 64) return LLMQ_ERR_SHAPE;
    // K slices of the few-token kernel: 1, 2, 4 (v = 0 or 8 .. 11); wavefronts along K of the streaming kernel: 4, 8
    const bool few = v == 0 || v >= 8;
    if (k_waves != 0 && !(k_waves == 4 || (few && (k_waves == 1 || k_waves == 2)) || (!few && k_waves == 8))) return LLMQ_ERR_SHAPE;
    set_awq_tile_direct_loads(staged ? 0 : 1);  // state changes only once the arguments are accepted
    g_force_v = v;
    g_force_splits = splits;
    g_force_kw = k_waves;
    return LLMQ_OK;
}

extern "C" size_t llmq_awq_gemm_workspace_bytes(int64_t M, int64_t N, int64_t K) {
    if (M <= 0 || N <= 0 || K <= 0) return 0;
    size_t total = 0;
    if (tile_path(M)) {
        const AwqTilePlan t = tile_plan(M, N, K);
        if (t.splits > 1) total = (size_t)t.splits * M * N * sizeof(float);
    }
    if (awq_decode_supported(M, N, K, 128)) {
        const size_t need = awq_decode_workspace_bytes(decode16_plan(M, N, K), M, N);
        if (need > total) total = need;
    }
    for (int64_t m0 = 0; m0 < M; m0 += 64) {
        const int64_t mm = M - m0 < 64 ? M - m0 : 64;
        const AwqPlan p = make_awq_plan(mm, N, K);  // sized for either kernel (the group size is not known here)
        size_t need = p.splits > 1 ? (size_t)p.splits * mm * N * sizeof(float) : 0;
        if (K % 128 == 0) {
            const DecodePlan d = make_decode_plan(mm, N, K);
            const size_t need2 = d.splits > 1 ? (size_t)d.splits * mm * N * sizeof(float) : 0;
            if (need2 > need) need = need2;
        }
        if (need > total) total = need;
    }
    return total ? kAwqTicketBytes + total : 0;  // the arrival counters come first
}

extern "C" size_t llmq_awq_workspace_ticket_bytes(void) { return kAwqTicketBytes; }

extern "C" int llmq_awq_workspace_init(void* workspace, size_t workspace_bytes, llmq_stream_t stream) {
    if (!workspace || workspace_bytes == 0) return LLMQ_OK;
    if (reinterpret_cast<uintptr_t>(workspace) & 15u) return LLMQ_ERR_ALIGN;
    return awq_clear_tickets(workspace, workspace_bytes, (hipStream_t)stream);
}

extern "C" int llmq_awq_gemm(const void* x, int64_t ldx, const int32_t* qweight, const void* scales,
                             const int32_t* qzeros, const void* bias, void* out, int64_t M, int64_t N, int64_t K,
                             int64_t group, void* workspace, size_t workspace_bytes, llmq_stream_t stream) {
    if (M < 0 || N < 0 || K < 0) return LLMQ_ERR_SHAPE;
    if (M == 0 || N == 0) return LLMQ_OK;
    if (!x || !qweight || !scales || !qzeros || !out) return LLMQ_ERR_NULL;
    if (K == 0 || (K % kChunkK) || (N & 7) || group <= 0 || (K % group) || (group % kChunkK) || ldx < K || (ldx & 7))
        return LLMQ_ERR_SHAPE;
    if (N > 0x7fffffffLL || K > 0x7fffffffLL || M > 0x7fffffffLL || ldx * 16 > 0x7fffffffLL) return LLMQ_ERR_SHAPE;
    if (!aligned16(x) || !aligned16(scales) || !aligned16(out) || (reinterpret_cast<uintptr_t>(qweight) & 15u) ||
        (reinterpret_cast<uintptr_t>(qzeros) & 15u) || (reinterpret_cast<uintptr_t>(workspace) & 15u))
        return LLMQ_ERR_ALIGN;
    hipStream_t st = (hipStream_t)stream;
    // workspace = arrival counters (kAwqTicketBytes, zero between calls), then partial sums (contents irrelevant)
    unsigned int* tickets = workspace_bytes > kAwqTicketBytes ? (unsigned int*)workspace : nullptr;
    float* ws = tickets ? (float*)((unsigned char*)workspace + kAwqTicketBytes) : nullptr;
    workspace_bytes = tickets ? workspace_bytes - kAwqTicketBytes : 0;
    const uint32_t* qw = (const uint32_t*)qweight;
    const uint32_t* qz = (const uint32_t*)qzeros;
    const uint16_t* sc = (const uint16_t*)scales;
    const uint16_t* bs = (const uint16_t*)bias;
    const int Ni = (int)N, Ki = (int)K, Gi = (int)group;
    if (tile_path(M)) {
        const AwqTilePlan t = tile_plan(M, N, K);
        if (t.splits > 1 && (!ws || workspace_bytes < (size_t)t.splits * M * N * sizeof(float))) return LLMQ_ERR_WORKSPACE;
        const int rc = launch_awq_tile(t, (const uint16_t*)x, ldx, qw, sc, qz, bs, (uint16_t*)out, ws, (int)M, Ni, Ki, Gi, st);
        if (rc != LLMQ_OK) return rc;
        if (t.splits > 1) {
            const int64_t total = M * N;
            const int blocks = (int)((total + 255) / 256 < 2048 ? (total + 255) / 256 : 2048);
            hipLaunchKernelGGL(awq_finish_kernel, dim3(blocks), dim3(256), 0, st, ws, t.splits, total, Ni, bs,
                               (uint16_t*)out);
            if (launch_status() != LLMQ_OK) return LLMQ_ERR_LAUNCH;
        }
        return LLMQ_OK;
    }
    if (decode16_path(M, N, K, group)) {
        const AwqDecodePlan d = decode16_plan(M, N, K);
        if (d.splits > 1 && (!ws || workspace_bytes < awq_decode_workspace_bytes(d, M, N))) return LLMQ_ERR_WORKSPACE;
        return launch_awq_decode(d, (const uint16_t*)x, ldx, qw, sc, qz, bs, (uint16_t*)out, tickets, ws, (int)M, Ni, Ki, st);
    }
    // tokens are processed in slabs of at most 64 rows (4 MFMA token tiles per weight pass)
    for (int64_t m0 = 0; m0 < M; m0 += 64) {
        const int mm = (int)(M - m0 < 64 ? M - m0 : 64);
        const uint16_t* xs = (const uint16_t*)x + m0 * ldx;
        uint16_t* os = (uint16_t*)out + m0 * N;
        int splits;
        if (decode_path(mm, group)) {
            const DecodePlan d = make_decode_plan(mm, N, K);
            splits = d.splits;
            if (splits > 1 && (!ws || workspace_bytes < (size_t)splits * mm * N * sizeof(float))) return LLMQ_ERR_WORKSPACE;
            const int ms = d.ms;
            const int slabs = cdiv(mm, 16 * ms);
            const dim3 grid(cdiv(Ni / 8, 16 * d.v) * slabs, splits);
#define LLMQ_AWQ_DECODE(VV, KWW, MSS) \
    hipLaunchKernelGGL((awq_gemv_kernel<VV, KWW, MSS>), grid, dim3(KWW * kWave), 0, st, xs, ldx, qw, sc, qz, bs, os, ws, mm, \
                       Ni, Ki, slabs)
            if (ms == 4) LLMQ_AWQ_DECODE(1, 4, 4);
            else if (ms == 2) LLMQ_AWQ_DECODE(1, 4, 2);
            else if (d.v == 2) LLMQ_AWQ_DECODE(2, 4, 1);
            else if (d.kw == 8) LLMQ_AWQ_DECODE(1, 8, 1);
            else LLMQ_AWQ_DECODE(1, 4, 1);
#undef LLMQ_AWQ_DECODE
        } else {
            const AwqPlan p = make_awq_plan(mm, N, K);
            splits = p.splits;
            if (splits > 1 && (!ws || workspace_bytes < (size_t)splits * mm * N * sizeof(float))) return LLMQ_ERR_WORKSPACE;
            if (p.mt == 1 && p.v == 2) launch_awq<2, 1>(p, xs, ldx, qw, sc, qz, bs, os, ws, mm, Ni, Ki, Gi, st);
            else if (p.mt == 1) launch_awq<1, 1>(p, xs, ldx, qw, sc, qz, bs, os, ws, mm, Ni, Ki, Gi, st);
            else if (p.mt == 2) launch_awq<1, 2>(p, xs, ldx, qw, sc, qz, bs, os, ws, mm, Ni, Ki, Gi, st);
            else launch_awq<1, 4>(p, xs, ldx, qw, sc, qz, bs, os, ws, mm, Ni, Ki, Gi, st);
        }
        if (launch_status() != LLMQ_OK) return LLMQ_ERR_LAUNCH;
        if (splits > 1) {
            const int64_t total = (int64_t)mm * N;
            const int blocks = (int)((total + 255) / 256 < 2048 ? (total + 255) / 256 : 2048);
            hipLaunchKernelGGL(awq_finish_kernel, dim3(blocks), dim3(256), 0, st, ws, splits, total, Ni, bs, os);
            if (launch_status() != LLMQ_OK) return LLMQ_ERR_LAUNCH;
        }
    }
    return LLMQ_OK;
}

extern "C" int llmq_awq_dequant(const int32_t* qweight, const void* scales, const int32_t* qzeros, void* out,
                                int64_t K, int64_t N, int64_t group, llmq_stream_t stream) {
    if (K < 0 || N < 0) return LLMQ_ERR_SHAPE;
    if (K == 0 || N == 0) return LLMQ_OK;
    if (!qweight || !scales || !qzeros || !out) return LLMQ_ERR_NULL;
    if ((N & 7) || group <= 0 || (K % group) || N > 0x7fffffffLL) return LLMQ_ERR_SHAPE;
    if (!aligned16(scales) || !aligned16(out)) return LLMQ_ERR_ALIGN;
    const int64_t total = K * (N / 8);
    if (group % 8 == 0 && K <= 0x7fffffffLL && (K / 8 + 3) / 4 <= 65535) {
        const dim3 grid((unsigned)((N / 8 + kWave - 1) / kWave), (unsigned)((K / 8 + 3) / 4));
        hipLaunchKernelGGL(awq_dequant_rows_kernel, grid, dim3(256), 0, (hipStream_t)stream, (const uint32_t*)qweight,
                           (const uint16_t*)scales, (const uint32_t*)qzeros, (uint16_t*)out, (int)K, (int)(N / 8),
                           (int)group);
        return launch_status();
    }
    const int blocks = (int)((total + 255) / 256 < 65536 ? (total + 255) / 256 : 65536);
    hipLaunchKernelGGL(awq_dequant_kernel, dim3(blocks), dim3(256), 0, (hipStream_t)stream, (const uint32_t*)qweight,
                       (const uint16_t*)scales, (const uint32_t*)qzeros, (uint16_t*)out, K, (int)(N / 8), (int)group);
    return launch_status();
}

extern "C" int llmq_awq_dequant_t(const int32_t* qweight, const void* scales, const int32_t* qzeros, void* out,
                                  int64_t K, int64_t N, int64_t group, llmq_stream_t stream) {
    if (K < 0 || N < 0) return LLMQ_ERR_SHAPE;
    if (K == 0 || N == 0) return LLMQ_OK;
    if (!qweight || !scales || !qzeros || !out) return LLMQ_ERR_NULL;
    if ((N & 7) || group <= 0 || (K % group) || (group & 7) || N > 0x7fffffffLL || K > 0x7fffffffLL || (K + 63) / 64 > 65535)
        return LLMQ_ERR_SHAPE;
    if (!aligned16(scales) || !aligned16(out)) return LLMQ_ERR_ALIGN;
    const dim3 grid((unsigned)((N / 8 + 31) / 32), (unsigned)((K + 63) / 64));
    hipLaunchKernelGGL(awq_dequant_t_kernel, grid, dim3(256), 0, (hipStream_t)stream, (const uint32_t*)qweight,
                       (const uint16_t*)scales, (const uint32_t*)qzeros, (uint16_t*)out, (int)K, (int)(N / 8), (int)group);
    return launch_status();
}
