// Few-token quantized linear in one launch: per-token dynamic activation quantizer + W8A8 int8 / FP8 GEMM +
// per-token x per-channel epilogue, for up to 16 tokens (decode).
//
//   s[m]    = round_dt( max(absmax_k |x[m,k]|, round_dt(floor)) / qmax )            the row quantizers of quant.hip
//   q[m,k]  = narrow( clamp( round_dt( x[m,k] / s[m] ) ) )
//   out     = ((sum_k q[m,k] * B[n,k]) * s[m]) * sw[n] + bias[n]                     llmq_gemm_w8a8 / llmq_gemm_fp8
//
// The reference runs these as separate steps (nn_models/modules/linear/linear_sq.py:97-138: the quantizer of
// lines 55-65, then the GEMM op; linear_fp8.py:40-63 + 199-221).  With a few tokens each step is a launch of a
// few microseconds that mostly waits; here the GEMM kernel quantizes its own activation operand:
//   * a block owns 16*T output channels, its NW wavefronts own consecutive runs of K steps, and the weights stream
//     from global memory straight into MFMA operand registers, exactly as in gemm_skinny.hip;
//   * before its first step a block quantizes the activations itself, once, into LDS: wavefront w takes tokens w,
//     w + NW, .., keeps the row in registers, reduces |x|, and writes the codes as the [token][K] int8 / fp8 matrix
//     the MFMA operand reads expect (the activations are a few KB per token and sit in L2; every block repeats this,
//     which is cheaper than a launch).  The first batch of weight loads is already in flight meanwhile;
//   * the arithmetic is the row quantizer's (quant_math.h), so codes and scales are bit-identical to
//     llmq_quant_*_per_token and the result is bit-identical to the two-launch form.  Block 0 can write codes and
//     scales out for checking.
// The quantized activations must fit in LDS: M * (K + 16) <= 64 KB (16 tokens at K = 3584, 3 at K = 18944).
// Measured on MI355X (Qwen2-7B projections, weights out of HBM, launches back to back): level with the quantizer +
// few-token GEMM pair at 1-3 tokens and K = 3584 (qkv 10.0 against 9.5 us, o 7.9 against 8.1, gate_up 32.5 against
// 34.5), slower at 16 tokens (16 against 11) and for K = 18944 (30 against 20): the stream hides a second launch, while
// the quantizer's load -> reduce -> quantize chain now precedes every block's first MFMA.  What it saves is a launch on
// the host side.  (Quantizing in the operand registers of every wavefront instead of once per block was measured
// 40-100 % slower: 15 of 16 MFMA rows repeat the same token's work at one token.)
#include <algorithm>
#include <type_traits>

#include "llmq_common.h"
#include "quant_math.h"

namespace llmq {
namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v8i __attribute__((ext_vector_type(8)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef uint32_t u4 __attribute__((ext_vector_type(4)));

struct FusedArgs {
    const uint16_t* x;       // [M, K] activations, row stride ldx elements
    const uint8_t* B;        // [N, K] quantized weights, row stride ldb bytes
    const float* w_scale;    // [N] or null
    const void* bias;        // [N] or null
    void* out;               // [M, N]
    uint8_t* q_dump;         // [M, K] quantized activations, or null
    float* scale_dump;       // [M] activation scales, or null
    void* acc_dump;          // [M, N] raw accumulators, or null
    int64_t ldx, ldb, ldo;
    int M, N, K;
    int bias_dtype, out_dtype;
};

constexpr int kRowPad = 16;        // bytes between LDS rows beyond K: consecutive tokens start 4 banks apart
constexpr int kMaxLdsBytes = 65536 - 256;
constexpr int kRowChunks = 10;     // 16-byte pieces of a row a lane keeps in registers (K <= 10 * 64 * 8 = 5120); longer rows are re-read

template <bool FP8, int DT, int T, int NW, int D>
__global__ __launch_bounds__(NW * kWave) void linear_fused_kernel(FusedArgs a) {
    constexpr int MODE = FP8 ? MODE_F8 : MODE_I8;
    constexpr int NT = NW * kWave, KSTEP = FP8 ? 128 : 64, P = FP8 ? 2 : 1, LB = 16 * P;  // LB codes per lane and step
    using acc_t = typename std::conditional<FP8, v4f, v4i>::type;
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];  // [M][K + kRowPad] codes; after the main loop: red[NW][T][64]
    __shared__ float s_scale[16];

    const int tid = threadIdx.x, lane = tid & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
    const int r16 = lane & 15, kq = lane >> 4;
    const int M = a.M, N = a.N, K = a.K;
    const int n0 = blockIdx.x * (16 * T);
    const int steps = (K + KSTEP - 1) / KSTEP, spw = (steps + NW - 1) / NW;
    const int s_begin = min(steps, wave * spw), s_end = min(steps, s_begin + spw);
    const int row_bytes = K + kRowPad;

    const uint8_t* pb[T];
#pragma unroll
    for (int t = 0; t < T; t++) pb[t] = a.B + (int64_t)min(n0 + 16 * t + r16, N - 1) * a.ldb + kq * LB;

    struct Batch { u4 b[D][T][P]; };
    // K % 16 == 0: a lane's 16-byte pieces are either inside K or past it; a piece past the end re-reads the row's
    // first bytes and is masked when it is used
    auto load_batch = [&](int s0, Batch& d) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < D; i++) {
            const int s = min(s0 + i, s_end - 1);
#pragma unroll
            for (int p = 0; p < P; p++) {
                const int koff = s * KSTEP + kq * LB + 16 * p;
                const int kc = koff < K ? s * KSTEP + 16 * p : -(kq * LB);
#pragma unroll
                for (int t = 0; t < T; t++) d.b[i][t][p] = *reinterpret_cast<const u4*>(pb[t] + kc);
            }
        }
    };

    Batch ba, bb;
    if (s_begin < s_end) load_batch(s_begin, ba);  // weights start streaming before the activations are quantized

    // ---- quantize: wavefront w takes tokens w, w + NW, ...; a lane owns the 16-byte pieces lane, lane + 64, ...
    const int nchunk = K >> 3;
    for (int m = wave; m < M; m += NW) {
        const uint4* row = reinterpret_cast<const uint4*>(a.x + (int64_t)m * a.ldx);
        uint4 cache[kRowChunks];
        float amax = 0.f;
#pragma unroll
        for (int c = 0; c < kRowChunks; c++) {
            const int i = lane + c * kWave;
            cache[c] = i < nchunk ? row[i] : make_uint4(0, 0, 0, 0);
        }
#pragma unroll
        for (int c = 0; c < kRowChunks; c++) amax = max_nonneg(amax, absmax8(cache[c], DT == LLMQ_BF16));
        for (int i = lane + kRowChunks * kWave; i < nchunk; i += kWave) amax = max_nonneg(amax, absmax8(row[i], DT == LLMQ_BF16));
        amax = wave_max(amax);
        const float s = scale_from_amax<DT, MODE>(amax), inv_s = 1.0f / s;
        if (lane == 0) {
            s_scale[m] = s;
            if (a.scale_dump && blockIdx.x == 0) a.scale_dump[m] = s;
        }
        uint2* qrow = reinterpret_cast<uint2*>(smem + m * row_bytes);
        uint2* qdump = (a.q_dump && blockIdx.x == 0) ? reinterpret_cast<uint2*>(a.q_dump + (int64_t)m * K) : nullptr;
#pragma unroll
        for (int c = 0; c < kRowChunks; c++) {
            const int i = lane + c * kWave;
            if (i < nchunk) {
                const uint2 q = quant8<DT, MODE, Q_DT>(cache[c], s, inv_s);
                qrow[i] = q;
                if (qdump) qdump[i] = q;
            }
        }
        for (int i = lane + kRowChunks * kWave; i < nchunk; i += kWave) {
            const uint2 q = quant8<DT, MODE, Q_DT>(row[i], s, inv_s);
            qrow[i] = q;
            if (qdump) qdump[i] = q;
        }
    }
    __syncthreads();
    const uint8_t* arow = smem + min(r16, M - 1) * row_bytes + kq * LB;  // rows past M repeat the last token; never stored

    acc_t acc[T];
#pragma unroll
    for (int t = 0; t < T; t++) acc[t] = acc_t{0, 0, 0, 0};

    auto compute_batch = [&](int s0, const Batch& d) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < D; i++) {
            const bool live = s0 + i < s_end;  // wavefront-uniform: steps past the run contribute nothing
            u4 bm[T][P], am[P];
#pragma unroll
            for (int p = 0; p < P; p++) {
                const int koff = (s0 + i) * KSTEP + kq * LB + 16 * p;
                const bool ok = live && koff < K;
                const uint32_t keep = ok ? 0xffffffffu : 0u;
#pragma unroll
                for (int t = 0; t < T; t++) bm[t][p] = d.b[i][t][p] & keep;
                am[p] = *reinterpret_cast<const u4*>(arow + (ok ? (s0 + i) * KSTEP + 16 * p : -(kq * LB)));
            }
#pragma unroll
            for (int t = 0; t < T; t++) {
                if constexpr (FP8) {
                    const v8i bw = {(int)bm[t][0][0], (int)bm[t][0][1], (int)bm[t][0][2], (int)bm[t][0][3],
                                    (int)bm[t][1][0], (int)bm[t][1][1], (int)bm[t][1][2], (int)bm[t][1][3]};
                    const v8i aw = {(int)am[0][0], (int)am[0][1], (int)am[0][2], (int)am[0][3],
                                    (int)am[1][0], (int)am[1][1], (int)am[1][2], (int)am[1][3]};
                    acc[t] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(bw, aw, acc[t], 0, 0, 0, 0, 0, 0);
                } else {
                    const v4i bw = {(int)bm[t][0][0], (int)bm[t][0][1], (int)bm[t][0][2], (int)bm[t][0][3]};
                    const v4i aw = {(int)am[0][0], (int)am[0][1], (int)am[0][2], (int)am[0][3]};
                    acc[t] = __builtin_amdgcn_mfma_i32_16x16x64_i8(bw, aw, acc[t], 0, 0, 0);
                }
            }
        }
    };

    if (s_begin < s_end) {
#pragma unroll 1
        for (int s = s_begin; s < s_end; s += 2 * D) {
            load_batch(s + D, bb);
            compute_batch(s, ba);
            load_batch(s + 2 * D, ba);
            compute_batch(s + D, bb);
        }
    }

    // ---- the block's wavefronts add up in wavefront order (int32: exact; fp32: fixed order)
    __syncthreads();  // every wavefront is done reading the codes: their memory is reused
    acc_t (*red)[T][kWave] = reinterpret_cast<acc_t (*)[T][kWave]>(smem);
#pragma unroll
    for (int t = 0; t < T; t++) red[wave][t][lane] = acc[t];
    __syncthreads();
    for (int idx = tid; idx < T * kWave; idx += NT) {
        const int t = idx / kWave, l = idx % kWave;
        acc_t sum = red[0][t][l];
#pragma unroll
        for (int w = 1; w < NW; w++) sum += red[w][t][l];
        // lane l of that accumulator: token l % 16, channels n0 + 16 t + 4 (l / 16) .. + 3
        const int m = l & 15, n = n0 + 16 * t + 4 * (l >> 4);
        if (m >= M || n >= N) continue;
        const float sa = s_scale[m];
        uint16_t h[4];
#pragma unroll
        for (int e = 0; e < 4; e++) {
            const int ne = min(n + e, N - 1);
            const float sw = a.w_scale ? a.w_scale[ne] : 1.f;
            const float bb2 = a.bias ? load_as_f32(a.bias, a.bias_dtype, ne) : 0.f;
            const float v = epi_value((float)sum[e], sa, sw, 1.0f, bb2);
            h[e] = a.out_dtype == LLMQ_BF16 ? Lo<LLMQ_BF16>::from_f32(v) : Lo<LLMQ_F16>::from_f32(v);
        }
        uint16_t* orow = reinterpret_cast<uint16_t*>(a.out) + (int64_t)m * a.ldo + n;
        if (n + 3 < N && ((reinterpret_cast<uintptr_t>(orow) & 7u) == 0)) {
            *reinterpret_cast<uint2*>(orow) = make_uint2((uint32_t)h[0] | ((uint32_t)h[1] << 16), (uint32_t)h[2] | ((uint32_t)h[3] << 16));
        } else {
#pragma unroll
            for (int e = 0; e < 4; e++)
                if (n + e < N) orow[e] = h[e];
        }
        if (a.acc_dump) {
#pragma unroll
            for (int e = 0; e < 4; e++)
                if (n + e < N) {
                    const auto sv = sum[e];  // scalar copy first: a bit cast applied to the vector element itself reads element 0
                    reinterpret_cast<uint32_t*>(a.acc_dump)[(int64_t)m * N + n + e] = __builtin_bit_cast(uint32_t, sv);
                }
        }
    }
}

thread_local int g_force_fused_variant = -1;  // tuning hook (per host thread): 0 = 2 channel tiles x 4 wavefronts, 1 = 1 x 8

template <bool FP8, int DT>
int launch_fused(const FusedArgs& a, hipStream_t st) {
    constexpr int D = FP8 ? 2 : 4;  // steps per batch: ~64 registers per batch
    // same split as the few-token GEMM: short K and many channels -> wider channel tiles, otherwise more wavefronts along K
    bool wide = a.K < 8192 && a.N >= 4096;
    if (g_force_fused_variant >= 0) wide = g_force_fused_variant == 0;
    const size_t lds = std::max<size_t>((size_t)a.M * (a.K + kRowPad), (size_t)8 * 1 * kWave * 16);  // codes, then the reduction
    if (wide) {
        hipLaunchKernelGGL((linear_fused_kernel<FP8, DT, 2, 4, D>), dim3((a.N + 31) / 32), dim3(4 * kWave), lds, st, a);
    } else {
        hipLaunchKernelGGL((linear_fused_kernel<FP8, DT, 1, 8, D>), dim3((a.N + 15) / 16), dim3(8 * kWave), lds, st, a);
    }
    return launch_status();
}

int fused_entry(bool fp8, const void* x, int x_dtype, int64_t ldx, const uint8_t* B, int64_t ldb, const float* w_scale,
                const void* bias, int bias_dtype, void* out, int out_dtype, int64_t ldo, int64_t M, int64_t N, int64_t K,
                uint8_t* q_dump, float* scale_dump, void* acc_dump, hipStream_t st) {
    if (M < 0 || N < 0 || K < 0) return LLMQ_ERR_SHAPE;
    if (M > 16 || M * (K + kRowPad) > kMaxLdsBytes) return LLMQ_ERR_SHAPE;  // llmq_linear_dynamic_max_tokens(K)
    if (M == 0 || N == 0) return LLMQ_OK;
    if (!x || !B || !out) return LLMQ_ERR_NULL;
    if (x_dtype != LLMQ_BF16 && x_dtype != LLMQ_F16) return LLMQ_ERR_DTYPE;
    if (out_dtype != LLMQ_BF16 && out_dtype != LLMQ_F16) return LLMQ_ERR_DTYPE;
    if (bias && bias_dtype != LLMQ_BF16 && bias_dtype != LLMQ_F16 && bias_dtype != LLMQ_F32) return LLMQ_ERR_DTYPE;
    if (K == 0 || (K & 15) || (ldx & 7) || (ldb & 15) || ldx < K || ldb < K || ldo < N) return LLMQ_ERR_SHAPE;
    if (N > 0x7fffffffLL || K > 0x7fffffffLL || ldx >= (1 << 22) || ldb >= (1 << 22)) return LLMQ_ERR_SHAPE;
    if (!aligned16(x) || !aligned16(B) || (q_dump && !aligned16(q_dump))) return LLMQ_ERR_ALIGN;
    const FusedArgs a{(const uint16_t*)x, B, w_scale, bias, out, q_dump, scale_dump, acc_dump, ldx, ldb, ldo,
                      (int)M, (int)N, (int)K, bias_dtype, out_dtype};
    if (fp8) return x_dtype == LLMQ_BF16 ? launch_fused<true, LLMQ_BF16>(a, st) : launch_fused<true, LLMQ_F16>(a, st);
    return x_dtype == LLMQ_BF16 ? launch_fused<false, LLMQ_BF16>(a, st) : launch_fused<false, LLMQ_F16>(a, st);
}

}  // namespace
}  // namespace llmq

using namespace llmq;

extern "C" int llmq_linear_dynamic_max_tokens(int64_t K) {
    if (K <= 0) return 0;
    const int64_t fit = kMaxLdsBytes / (K + kRowPad);
    return (int)(fit < 16 ? fit : 16);
}

extern "C" int llmq_linear_dynamic_force_variant(int v) {
    if (v < -1 || v > 1) return LLMQ_ERR_SHAPE;
    g_force_fused_variant = v;
    return LLMQ_OK;
}

extern "C" int llmq_linear_i8_dynamic(const void* x, int x_dtype, int64_t ldx, const int8_t* B, int64_t ldb,
                                      const float* w_scale, const void* bias, int bias_dtype, void* out, int out_dtype,
                                      int64_t ldo, int64_t M, int64_t N, int64_t K, int8_t* q_dump, float* scale_dump,
                                      int32_t* acc_dump, llmq_stream_t stream) {
    return fused_entry(false, x, x_dtype, ldx, (const uint8_t*)B, ldb, w_scale, bias, bias_dtype, out, out_dtype, ldo, M, N, K,
                       (uint8_t*)q_dump, scale_dump, acc_dump, (hipStream_t)stream);
}

extern "C" int llmq_linear_fp8_dynamic(const void* x, int x_dtype, int64_t ldx, const uint8_t* B, int64_t ldb,
                                       const float* w_scale, const void* bias, int bias_dtype, void* out, int out_dtype,
                                       int64_t ldo, int64_t M, int64_t N, int64_t K, uint8_t* q_dump, float* scale_dump,
                                       float* acc_dump, llmq_stream_t stream) {
    return fused_entry(true, x, x_dtype, ldx, B, ldb, w_scale, bias, bias_dtype, out, out_dtype, ldo, M, N, K, q_dump,
                       scale_dump, acc_dump, (hipStream_t)stream);
}
