// W8A8 int8 / FP8 GEMM for a few tokens (M <= 64): one launch, no LDS staging, no workspace.
//
//   acc[m,n] = sum_k A[m,k] * B[n,k]        A: [M,K] row-major, B: [N,K] row-major (both K-contiguous)
//
// With at most 64 tokens the op streams the weights once out of HBM (M*K + N*K bytes for 2*M*N*K operations) and
// the matrix cores idle; what counts is bytes in flight and a short instruction stream.  Both operands are
// K-contiguous, and that is the layout a lane of the 16x16 MFMAs wants (lane (r, kq) feeds 16 or 32 consecutive
// K-bytes of row r), so the weights go from global memory straight into the operand registers:
//   * a block owns 16*T output channels, its NW wavefronts own consecutive runs of K steps (64 bytes of K for
//     v_mfma_i32_16x16x64_i8, 128 for v_mfma_f32_16x16x128_f8f6f4).  A wavefront load instruction fetches 16 rows x
//     64 (128) bytes; consecutive steps continue the same rows, so both halves of every 128-byte line are requested
//     back to back by the same wavefront.
//   * loads are issued in batches of D steps into one of two register sets; the next batch is in flight while the
//     current one feeds the matrix cores (branch-free: a step past the run re-reads its last one, bytes past the
//     ragged end of K are masked to zero).
//   * the weights are the MFMA row operand, so a lane ends up with 4 consecutive channels of one token.  The
//     wavefronts of a block add their accumulators through LDS in wavefront order (int32: exact; fp32: fixed order,
//     deterministic), and the block applies the same epilogue as the tile kernel and stores 8 bytes per lane.
#include <type_traits>

#include "llmq_common.h"

namespace llmq {

struct SkinnyEpilogue {
    const float* a_scale;    // [M] or null
    const float* w_scale;    // [N] or null
    const float* alpha_dev;  // device scalar or null
    const void* bias;        // [N] or null
    float alpha, beta;
    int bias_dtype, out_dtype;
};

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v8i __attribute__((ext_vector_type(8)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef uint32_t u4 __attribute__((ext_vector_type(4)));

template <bool FP8, int AFMT, int MT, int T, int NW, int D>
__global__ __launch_bounds__(NW * kWave) void gemm_skinny_kernel(
    const uint8_t* __restrict__ A, int64_t lda, const uint8_t* __restrict__ B, int64_t ldb, int M, int N, int K,
    SkinnyEpilogue ep, void* __restrict__ out, int64_t ldo, void* __restrict__ acc_dump) {
    constexpr int NT = NW * kWave, KSTEP = FP8 ? 128 : 64, P = FP8 ? 2 : 1, LB = 16 * P;  // P 16-byte pieces per lane and operand
    using acc_t = typename std::conditional<FP8, v4f, v4i>::type;
    __shared__ __attribute__((aligned(16))) acc_t red[NW][MT * T][kWave];

    const int tid = threadIdx.x, lane = tid & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
    const int r16 = lane & 15, kq = lane >> 4;
    const int n0 = blockIdx.x * (16 * T);
    const int steps = (K + KSTEP - 1) / KSTEP, spw = (steps + NW - 1) / NW;
    const int s_begin = min(steps, wave * spw), s_end = min(steps, s_begin + spw);

    const uint8_t* pb[T];
    const uint8_t* pa[MT];
#pragma unroll
    for (int t = 0; t < T; t++) pb[t] = B + (int64_t)min(n0 + 16 * t + r16, N - 1) * ldb + kq * LB;
#pragma unroll
    for (int mt = 0; mt < MT; mt++) pa[mt] = A + (int64_t)min(16 * mt + r16, M - 1) * lda + kq * LB;

    struct Batch { u4 b[D][T][P], a[D][MT][P]; };
    // K % 16 == 0: a 16-byte piece is either whole or past the end; a piece past the end re-reads the row's first
    // bytes and is masked when it is used
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
#pragma unroll
                for (int mt = 0; mt < MT; mt++) d.a[i][mt][p] = *reinterpret_cast<const u4*>(pa[mt] + kc);
            }
        }
    };

    acc_t acc[MT][T];
#pragma unroll
    for (int mt = 0; mt < MT; mt++)
#pragma unroll
        for (int t = 0; t < T; t++) acc[mt][t] = acc_t{0, 0, 0, 0};

    auto compute_batch = [&](int s0, const Batch& d) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < D; i++) {
            const bool live = s0 + i < s_end;  // wavefront-uniform: steps past the run contribute nothing
            u4 bm[T][P];
#pragma unroll
            for (int p = 0; p < P; p++) {
                const int koff = (s0 + i) * KSTEP + kq * LB + 16 * p;
                const uint32_t keep = (live && koff < K) ? 0xffffffffu : 0u;
#pragma unroll
                for (int t = 0; t < T; t++) bm[t][p] = d.b[i][t][p] & keep;
            }
#pragma unroll
            for (int mt = 0; mt < MT; mt++)
#pragma unroll
                for (int t = 0; t < T; t++) {
                    if constexpr (FP8) {
                        const v8i bw = {(int)bm[t][0][0], (int)bm[t][0][1], (int)bm[t][0][2], (int)bm[t][0][3],
                                        (int)bm[t][1][0], (int)bm[t][1][1], (int)bm[t][1][2], (int)bm[t][1][3]};
                        const u4 a0 = d.a[i][mt][0], a1 = d.a[i][mt][1];
                        const v8i aw = {(int)a0[0], (int)a0[1], (int)a0[2], (int)a0[3], (int)a1[0], (int)a1[1], (int)a1[2], (int)a1[3]};
                        acc[mt][t] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(bw, aw, acc[mt][t], 0, AFMT, 0, 0, 0, 0);
                    } else {
                        const v4i bw = {(int)bm[t][0][0], (int)bm[t][0][1], (int)bm[t][0][2], (int)bm[t][0][3]};
                        const u4 a0 = d.a[i][mt][0];
                        const v4i aw = {(int)a0[0], (int)a0[1], (int)a0[2], (int)a0[3]};
                        acc[mt][t] = __builtin_amdgcn_mfma_i32_16x16x64_i8(bw, aw, acc[mt][t], 0, 0, 0);
                    }
                }
        }
    };

    if (s_begin < s_end) {
        Batch ba, bb;
        load_batch(s_begin, ba);
#pragma unroll 1
        for (int s = s_begin; s < s_end; s += 2 * D) {
            load_batch(s + D, bb);
            compute_batch(s, ba);
            load_batch(s + 2 * D, ba);
            compute_batch(s + D, bb);
        }
    }

    // ---- the block's wavefronts add up in wavefront order
#pragma unroll
    for (int mt = 0; mt < MT; mt++)
#pragma unroll
        for (int t = 0; t < T; t++) red[wave][mt * T + t][lane] = acc[mt][t];
    __syncthreads();
    const float alpha = ep.alpha * (ep.alpha_dev ? *ep.alpha_dev : 1.0f);
    for (int idx = tid; idx < MT * T * kWave; idx += NT) {
        const int q = idx / kWave, l = idx % kWave, mt = q / T, t = q % T;
        acc_t sum = red[0][q][l];
#pragma unroll
        for (int w = 1; w < NW; w++) sum += red[w][q][l];
        // lane l of that accumulator: token 16 mt + l % 16, channels n0 + 16 t + 4 (l / 16) .. + 3
        const int m = 16 * mt + (l & 15), n = n0 + 16 * t + 4 * (l >> 4);
        if (m >= M || n >= N) continue;
        const float sa = ep.a_scale ? ep.a_scale[m] : 1.f;
        uint16_t h[4];
#pragma unroll
        for (int e = 0; e < 4; e++) {
            const int ne = min(n + e, N - 1);
            const float sw = ep.w_scale ? ep.w_scale[ne] : 1.f;
            const float bb = ep.bias ? ep.beta * load_as_f32(ep.bias, ep.bias_dtype, ne) : 0.f;
            const float v = epi_value((float)sum[e], sa, sw, alpha, bb);
            h[e] = ep.out_dtype == LLMQ_BF16 ? Lo<LLMQ_BF16>::from_f32(v) : Lo<LLMQ_F16>::from_f32(v);
        }
        uint16_t* orow = reinterpret_cast<uint16_t*>(out) + (int64_t)m * ldo + n;
        if (n + 3 < N && ((reinterpret_cast<uintptr_t>(orow) & 7u) == 0)) {
            *reinterpret_cast<uint2*>(orow) = make_uint2((uint32_t)h[0] | ((uint32_t)h[1] << 16), (uint32_t)h[2] | ((uint32_t)h[3] << 16));
        } else {
#pragma unroll
            for (int e = 0; e < 4; e++)
                if (n + e < N) orow[e] = h[e];
        }
        if (acc_dump) {
#pragma unroll
            for (int e = 0; e < 4; e++)
                if (n + e < N) {
                    const auto sv = sum[e];  // scalar copy first: a bit cast applied to the vector element itself reads element 0
                    reinterpret_cast<uint32_t*>(acc_dump)[(int64_t)m * N + n + e] = __builtin_bit_cast(uint32_t, sv);
                }
        }
    }
}

template <bool FP8, int AFMT, int MT, int T, int NW>
void launch_skinny_d(const uint8_t* A, int64_t lda, const uint8_t* B, int64_t ldb, int M, int N, int K,
                     const SkinnyEpilogue& ep, void* out, int64_t ldo, void* acc_dump, hipStream_t st) {
    // steps per batch: about 96 to 128 registers for the two batches in flight
    constexpr int D = FP8 ? (MT == 4 ? 1 : 2) : (MT == 4 ? 2 : 4);
    const int blocks = (N + 16 * T - 1) / (16 * T);
    hipLaunchKernelGGL((gemm_skinny_kernel<FP8, AFMT, MT, T, NW, D>), dim3(blocks), dim3(NW * kWave), 0, st, A, lda, B, ldb, M,
                       N, K, ep, out, ldo, acc_dump);
}

template <bool FP8, int AFMT, int MT>
void launch_skinny_mt(int t, int nw, const uint8_t* A, int64_t lda, const uint8_t* B, int64_t ldb, int M, int N, int K,
                      const SkinnyEpilogue& ep, void* out, int64_t ldo, void* acc_dump, hipStream_t st) {
#define LLMQ_SK(T_, NW_) launch_skinny_d<FP8, AFMT, MT, T_, NW_>(A, lda, B, ldb, M, N, K, ep, out, ldo, acc_dump, st)
    if (t == 1) {
        if (nw == 4) LLMQ_SK(1, 4);
        else if (nw == 16) LLMQ_SK(1, 16);
        else LLMQ_SK(1, 8);
    } else {
        if (nw == 4) LLMQ_SK(2, 4);
        else if (nw == 16 && MT <= 2) LLMQ_SK(2, (MT <= 2 ? 16 : 8));
        else LLMQ_SK(2, 8);
    }
#undef LLMQ_SK
}

}  // namespace

bool gemm_skinny_supported(int64_t M) { return M >= 1 && M <= 64; }

// t: 16-channel tiles per wavefront (1 | 2), nw: wavefronts per block (4 | 8 | 16); a_format: 0 e4m3, 1 e5m2 (fp8 only)
int launch_gemm_skinny(bool fp8, int a_format, int t, int nw, const uint8_t* A, int64_t lda, const uint8_t* B, int64_t ldb,
                       int M, int N, int K, const SkinnyEpilogue& ep, void* out, int64_t ldo, void* acc_dump,
                       hipStream_t st) {
    const int mt = M <= 16 ? 1 : (M <= 32 ? 2 : 4);
#define LLMQ_SK_MT(FP8_, AF_)                                                                                       \
    do {                                                                                                            \
        if (mt == 1) launch_skinny_mt<FP8_, AF_, 1>(t, nw, A, lda, B, ldb, M, N, K, ep, out, ldo, acc_dump, st);      \
        else if (mt == 2) launch_skinny_mt<FP8_, AF_, 2>(t, nw, A, lda, B, ldb, M, N, K, ep, out, ldo, acc_dump, st); \
        else launch_skinny_mt<FP8_, AF_, 4>(t, nw, A, lda, B, ldb, M, N, K, ep, out, ldo, acc_dump, st);              \
    } while (0)
    if (!fp8) LLMQ_SK_MT(false, 0);
    else if (a_format == 0) LLMQ_SK_MT(true, 0);
    else LLMQ_SK_MT(true, 1);
#undef LLMQ_SK_MT
    return launch_status();
}

}  // namespace llmq
