// W8A8 int8, FP8 (OCP e4m3fn / e5m2) and fp16 GEMMs: the planner (tile configuration, K split, few-token kernel,
// tail split) and the C entry points.  The tile kernels live in gemm_tile_impl.h and are instantiated per operand
// format in gemm_tile_*.hip; the few-token kernel in gemm_skinny.hip.
#include <algorithm>
#include <type_traits>

#include "gemm_tile.h"
#include "llmq_common.h"

namespace llmq {

// Few-token kernel (gemm_skinny.hip): one launch, no workspace.
struct SkinnyEpilogue {
    const float* a_scale;
    const float* w_scale;
    const float* alpha_dev;
    const void* bias;
    float alpha, beta;
    int bias_dtype, out_dtype;
};
bool gemm_skinny_supported(int64_t M);
int launch_gemm_skinny(bool fp8, int a_format, int t, int nw, const uint8_t* A, int64_t lda, const uint8_t* B, int64_t ldb,
                       int M, int N, int K, const SkinnyEpilogue& ep, void* out, int64_t ldo, void* acc_dump,
                       hipStream_t st);

namespace {

// Tuning/diagnostic knob (llmq_gemm_force_plan): forces a tile configuration and K split.
thread_local int g_force_cfg = -1, g_force_splits = 1, g_force_dma = -1;  // per host thread; g_force_dma: 0 = register-staged loop only
bool plan_override(int& cfg, int& splits) {
    if (g_force_cfg < 0) return false;
    cfg = g_force_cfg;
    splits = g_force_splits;
    return true;
}

// Up to 64 tokens: the streaming kernel without LDS staging.  llmq_gemm_force_plan(100 + v, .) forces it with
// 1 + (v & 1) channel tiles per wavefront and 4 << (v >> 1) wavefronts per block; a forced tile configuration
// (cfg >= 0) keeps the tile kernel.
bool skinny_plan(int64_t M, int64_t N, int64_t K, int& t, int& nw) {
    if (!gemm_skinny_supported(M)) return false;
    if (g_force_cfg >= 100) {
        const int v = g_force_cfg - 100;
        t = 1 + (v & 1);
        nw = 4 << (v >> 1);
        return true;
    }
    if (g_force_cfg >= 0) return false;
    // Measured on the Qwen2-7B projections with the weights coming out of HBM, against the tile kernel (with and
    // without split K): ahead up to 16 tokens for every projection with N <= 8192 (8 tokens for a long K: every
    // wavefront re-reads the activations of its K run), and up to 32 tokens for a short K, where the tile kernel has
    // only N / 128 blocks to pull the weights with (o: 7.1 / 8.3 us against 14.0 / 13.1 at 17 / 32 tokens, qkv 9.4 /
    // 10.9 against 15.7 / 15.5); a narrow N keeps the lead to 64 tokens with 16 wavefronts along K (o: 11.3 against
    // 13.5 us).  For gate_up (N = 37888) the tile kernel already streams at 5.5 TB/s.
    if (N > 8192) return false;
    if (K >= 8192) {
        if (M > 8) return false;
        t = 1, nw = 8;
        return true;
    }
    if (M <= 16) {
        if (N >= 4096) t = 2, nw = 4;
        else t = 1, nw = 8;
        return true;
    }
    if (M <= 32) {
        t = N >= 4096 ? 2 : 1, nw = 4;
        return true;
    }
    if (N < 4096) {
        t = 1, nw = 16;
        return true;
    }
    return false;
}

// Pick the tile shape and K split with the smallest modelled time:
// waves of blocks over the CUs x per-block MFMA time, with a floor from the bytes each block streams.
// mfma_scale: matrix-core time per K byte relative to int8 / fp8 (fp16: 2)
// fp8: the 64-byte K tiles have one MFMA sub-step there and keep the register-staged loop (measured ~20 % slower)
Plan make_plan(int64_t M, int64_t N, int64_t K, double mfma_scale = 1.0, bool fp8 = false) {
    int ocfg, osp;
    if (plan_override(ocfg, osp) && ocfg < 100) {
        const TileShape s = kShapes[ocfg < kNumShapes ? ocfg : kNumShapes - 1];
        const int kps = cdiv(cdiv(K, osp), s.bk) * s.bk;
        return Plan{ocfg < kNumShapes ? ocfg : kNumShapes - 1, cdiv(K, kps), kps};
    }
    // Cost model calibrated on MI355X (microseconds) with the direct-load kernels: a block needs t_tile per 64 bytes
    // of K plus a fixed prologue/epilogue cost; blocks execute in rounds over the 256 CUs (the small tiles are bound
    // by the CU's load path, so co-resident blocks share it and are not modelled as extra slots).  The chip is
    // power-limited under MFMA load: with a fraction f of the CUs busy a K tile takes (0.52 + 0.48 f) of its
    // full-chip time, so a partly filled round is cheaper than a full one.  Split-K adds a second kernel and the round
    // trip of the fp32/int32 partials.  Checked against a sweep of every configuration x K split at M = 128 / 512 /
    // 2048: the plan picked is within 1.5 % of the best measured one on average.
    struct Model { int cfg, per_cu; double t_tile, fixed; };
    static const Model kModels[] = {
        {1, 1, 0.88, 13.0},  // 256x256, 8 waves
        {2, 1, 0.60, 12.0},  // 256x128
        {3, 1, 0.27, 8.0},   // 128x128
        {4, 1, 0.17, 7.0},   // 64x128 (0.15 with its operands in the Infinity Cache; 0.17 is what it takes with weights out of HBM)
        {5, 1, 0.10, 6.0},   // 32x128
        {7, 1, 0.45, 8.0},   // 128x256, 8 waves
    };
    Plan best{1, 1, (int)K};
    double best_t = 1e300;
    for (const Model& md : kModels) {
        const TileShape s = kShapes[md.cfg];
        // skinny tiles are for small M; the 64-row tile also serves up to 1024 rows when 128x128 tiles
        // could not even fill the CUs once and K is short (measured: o and qkv at M = 512)
        if (M > 128 && md.cfg == 5) continue;
        if (M > 128 && md.cfg == 4 && (M > 1024 || (int64_t)cdiv(M, 128) * cdiv(N, 128) >= 2 * kNumCu)) continue;
        if (md.cfg < 5 && M <= s.bm / 2) continue;            // mostly padding
        // 128x256 tiles are for grids that 256x256 tiles cannot fill twice over (measured: o / down at M = 2048,
        // gate_up at M = 512, qkv at M = 4096: 8-17 % ahead; with more tiles the big tile's lower operand traffic wins)
        if (md.cfg == 7 && (M <= 64 || (int64_t)cdiv(M, 256) * cdiv(N, 256) >= 2 * kNumCu)) continue;
        const int64_t tiles = (int64_t)cdiv(M, s.bm) * cdiv(N, s.bn);
        for (int sp = 1; sp <= 16; sp++) {
            if (sp > 1 && (K / sp < 512 || (int64_t)M * N * sp > (int64_t)64 << 20)) break;
            const int kps = cdiv(cdiv(K, sp), s.bk) * s.bk;
            const int eff_sp = cdiv(K, kps);
            if (eff_sp != sp) continue;
            const int64_t slots = (int64_t)kNumCu * md.per_cu, blocks = tiles * sp;
            const int64_t full_rounds = blocks / slots, rest = blocks % slots;
            // fp8: the 64-byte K tiles run the slower register-staged loop; unsplit, config 1 is launched as the
            // 128-byte-tile config 6 (gemm_entry), which does not
            const double tt = md.t_tile * mfma_scale * (fp8 && s.bk == 64 && !(md.cfg == 1 && sp == 1) ? 1.2 : 1.0);
            double t = full_rounds * (kps / 64.0 * tt + md.fixed);
            if (rest) t += kps / 64.0 * tt * (0.52 + 0.48 * (double)rest / slots) + md.fixed;
            // two 64-row blocks fit a CU side by side and share its load path: between one and two blocks per CU the
            // launch is one stretched round, not two (measured: 288 blocks of K = 3584 take 20 us, 224 take 14)
            if (md.cfg == 4 && blocks > slots && blocks <= 2 * slots) t = kps / 64.0 * tt * blocks / slots + md.fixed + 3.0;
            if (sp > 1) t += 5.0 + (double)M * N * sp * 8.0 / 8.0e6;
            if (t < best_t) { best_t = t; best = Plan{md.cfg, sp, kps}; }
        }
    }
    return best;
}

// op: 0 int8, 1 fp8 (a_format picks the A format), 2 fp16 (K, lda, ldb in bytes, i.e. twice the element counts)
// out_scale (device scalar, may be null): out is fp32 [M, N] holding the out_dtype result after a round trip through
// e4m3fn on that scale (tile kernel's general epilogue; no few-token kernel, no tail split)
int gemm_entry(int op, int a_format, const uint8_t* A, int64_t lda, const uint8_t* B, int64_t ldb,
               const float* a_scale, const float* w_scale, float alpha, const float* alpha_dev, const void* bias,
               int bias_dtype, float beta, void* out, int out_dtype, int64_t ldo, int64_t M, int64_t N, int64_t K,
               void* acc_dump, void* ws, size_t ws_bytes, hipStream_t st, const float* out_scale = nullptr) {
    const bool fp8 = op == 1;
    if (M < 0 || N < 0 || K < 0) return LLMQ_ERR_SHAPE;
    if (M == 0 || N == 0) return LLMQ_OK;
    if (!A || !B || !out) return LLMQ_ERR_NULL;
    if (K == 0 || (K & 15) || (lda & 15) || (ldb & 15) || lda < K || ldb < K || ldo < N) return LLMQ_ERR_SHAPE;
    if (M > 0x7fffffffLL || N > 0x7fffffffLL || K > 0x7fffffffLL || lda >= (1 << 22) || ldb >= (1 << 22)) return LLMQ_ERR_SHAPE;
    if (out_dtype != LLMQ_BF16 && out_dtype != LLMQ_F16) return LLMQ_ERR_DTYPE;
    if (bias && bias_dtype != LLMQ_BF16 && bias_dtype != LLMQ_F16 && bias_dtype != LLMQ_F32) return LLMQ_ERR_DTYPE;
    if (fp8 && a_format != LLMQ_E4M3 && a_format != LLMQ_E5M2) return LLMQ_ERR_DTYPE;
    if (!aligned16(A) || !aligned16(B)) return LLMQ_ERR_ALIGN;
    int sk_t, sk_nw;
    if (op != 2 && !out_scale && skinny_plan(M, N, K, sk_t, sk_nw)) {
        const SkinnyEpilogue sep{a_scale, w_scale, alpha_dev, bias, alpha, beta, bias_dtype, out_dtype};
        return launch_gemm_skinny(fp8, a_format == LLMQ_E5M2 ? 1 : 0, sk_t, sk_nw, A, lda, B, ldb, (int)M, (int)N, (int)K, sep,
                                  out, ldo, acc_dump, st);
    }
    Plan p = make_plan(M, N, K, op == 2 ? 2.0 : 1.0, fp8);
    // fp8 fragments are twice as wide: the 8-wave prefill tile runs ~5 % faster with 128-byte K tiles
    if (fp8 && g_force_cfg < 0 && p.cfg == 1 && p.splits == 1) p.cfg = 6;
    // int8 with direct loads: no staging registers, so the 128-byte K tile fits (half the barriers, whole lines per row)
    if (!fp8 && g_force_cfg < 0 && p.cfg == 1 && K % 128 == 0 && p.k_per_split % 128 == 0) p.cfg = 6;
    if (p.splits > 1) {
        if (!ws || ws_bytes < (size_t)p.splits * M * N * 4) return LLMQ_ERR_WORKSPACE;
    }
    auto run = [&](const Plan& pl, const uint8_t* Bp, const float* wsc, const void* bs, void* o, int64_t n) {
        Epilogue ep{a_scale, wsc, alpha_dev, bs, alpha, beta, bias_dtype, out_dtype, out_scale};
        const bool dma = g_force_dma != 0;
        if (op == 2) return launch_gemm_f16(A, lda, Bp, ldb, (int)M, (int)n, (int)K, pl, ep, o, ldo, acc_dump, ws, dma, st);
        if (!fp8) return launch_gemm_i8(A, lda, Bp, ldb, (int)M, (int)n, (int)K, pl, ep, o, ldo, acc_dump, ws, dma, st);
        if (a_format == LLMQ_E4M3)
            return launch_gemm_fp8_e4m3(A, lda, Bp, ldb, (int)M, (int)n, (int)K, pl, ep, o, ldo, acc_dump, ws, dma, st);
        return launch_gemm_fp8_e5m2(A, lda, Bp, ldb, (int)M, (int)n, (int)K, pl, ep, o, ldo, acc_dump, ws, dma, st);
    };
    // Tail split.  When the 256x256 grid ends in a round that fills at most 5/8 of the CUs, the channels are cut at a
    // whole number of rounds: the first part keeps the big tiles and ends with every CU busy, the rest runs as one
    // round of 128x256 tiles (twice the blocks, half the time each).  Measured: 8192 x 4608 x 3584 (2.25 rounds)
    // and 8192 x 37888 x 3584 (18.5 rounds).
    if (g_force_cfg < 0 && p.cfg == 6 && p.splits == 1 && !acc_dump && !out_scale && K % 128 == 0) {
        const int64_t tm = cdiv(M, 256), tn = cdiv(N, 256), tiles = tm * tn, tail = tiles % kNumCu, full = tiles - tail;
        if (full >= kNumCu && tail > 0 && tail <= 160 && full % tm == 0) {
            const int64_t n1 = full / tm * 256, n2 = N - n1;
            if (n2 > 0 && (int64_t)cdiv(M, 128) * cdiv(n2, 256) <= kNumCu) {
                const int rc = run(p, B, w_scale, bias, out, n1);
                if (rc != LLMQ_OK) return rc;
                const int64_t be = bias_dtype == LLMQ_F32 ? 4 : 2;
                return run(Plan{7, 1, (int)K}, B + n1 * ldb, w_scale ? w_scale + n1 : nullptr,
                           bias ? static_cast<const uint8_t*>(bias) + n1 * be : nullptr, static_cast<uint8_t*>(out) + n1 * 2, n2);
            }
        }
    }
    return run(p, B, w_scale, bias, out, N);
}

// ---- scratch owned by the library, for the entry point that takes no workspace ---------------------
// One copy of this array exists on every GPU the library is loaded on, for the life of the process.
constexpr size_t kStaticScratchBytes = (size_t)32 << 20;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];
// `scratch` is a host-side stand-in for the symbol, not a device address: the address of each GPU's copy
// is looked up once per device and only that pointer is ever handed to a kernel.
void* g_scratch_ptr[64] = {};

int static_scratch(void** out) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return LLMQ_ERR_LAUNCH;
    if (!g_scratch_ptr[dev]) {
        void* p = nullptr;
        if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || !p) return LLMQ_ERR_LAUNCH;
        g_scratch_ptr[dev] = p;  // benign if two threads race here: both store the same address
    }
    *out = g_scratch_ptr[dev];
    return LLMQ_OK;
}

}  // namespace
}  // namespace llmq

using namespace llmq;

extern "C" size_t llmq_gemm_static_scratch_bytes(void) { return kStaticScratchBytes; }

extern "C" int llmq_gemm_w8a8_static(const int8_t* A, int64_t lda, const int8_t* B, int64_t ldb, const float* a_scale,
                                     const float* w_scale, float alpha, const float* alpha_dev, const void* bias,
                                     int bias_dtype, float beta, void* out, int out_dtype, int64_t ldo, int64_t M,
                                     int64_t N, int64_t K, llmq_stream_t stream) {
    void* ws = nullptr;
    int rc = static_scratch(&ws);
    if (rc != LLMQ_OK) return rc;
    // The common entry validates the arguments first and then checks the partial sums of the plan it is about to
    // launch (the int8 plan of this problem) against the size it is given: a plan that does not fit the array is
    // refused there, before any launch.
    rc = gemm_entry(0, 0, (const uint8_t*)A, lda, (const uint8_t*)B, ldb, a_scale, w_scale, alpha, alpha_dev, bias,
                    bias_dtype, beta, out, out_dtype, ldo, M, N, K, nullptr, ws, kStaticScratchBytes,
                    (hipStream_t)stream);
    return rc == LLMQ_ERR_WORKSPACE ? LLMQ_ERR_SCRATCH : rc;
}

extern "C" int llmq_gemm_force_plan(int cfg, int splits) {
    int dma = -1;
    if (cfg >= 0 && cfg < 100 && (cfg & 64)) dma = 0, cfg &= ~64;
    if ((cfg >= kNumShapes && (cfg < 100 || cfg > 105)) || splits < 1 || splits > 64) return LLMQ_ERR_SHAPE;
    g_force_dma = dma;
    g_force_cfg = cfg;
    g_force_splits = splits;
    return LLMQ_OK;
}

extern "C" int llmq_gemm_num_configs(void) { return kNumShapes; }

extern "C" size_t llmq_gemm_workspace_bytes(int64_t M, int64_t N, int64_t K) {
    if (M <= 0 || N <= 0 || K <= 0) return 0;
    int sk_t, sk_nw;
    if (skinny_plan(M, N, K, sk_t, sk_nw)) return 0;
    const Plan p = make_plan(M, N, K), p8 = make_plan(M, N, K, 1.0, true);  // the int8 and the fp8 plan may differ
    const int splits = p.splits > p8.splits ? p.splits : p8.splits;
    return splits > 1 ? (size_t)splits * M * N * 4 : 0;
}

extern "C" int llmq_gemm_w8a8(const int8_t* A, int64_t lda, const int8_t* B, int64_t ldb, const float* a_scale,
                              const float* w_scale, float alpha, const float* alpha_dev, const void* bias,
                              int bias_dtype, float beta, void* out, int out_dtype, int64_t ldo, int64_t M, int64_t N,
                              int64_t K, int32_t* acc_dump, void* workspace, size_t workspace_bytes,
                              llmq_stream_t stream) {
    return gemm_entry(0, 0, (const uint8_t*)A, lda, (const uint8_t*)B, ldb, a_scale, w_scale, alpha, alpha_dev,
                      bias, bias_dtype, beta, out, out_dtype, ldo, M, N, K, acc_dump, workspace, workspace_bytes,
                      (hipStream_t)stream);
}

extern "C" int llmq_gemm_fp8(const uint8_t* A, int a_format, int64_t lda, const uint8_t* B, int64_t ldb,
                             const float* a_scale, const float* w_scale, float alpha, const float* alpha_dev,
                             const void* bias, int bias_dtype, float beta, void* out, int out_dtype, int64_t ldo,
                             int64_t M, int64_t N, int64_t K, float* acc_dump, void* workspace,
                             size_t workspace_bytes, llmq_stream_t stream) {
    return gemm_entry(1, a_format, A, lda, B, ldb, a_scale, w_scale, alpha, alpha_dev, bias, bias_dtype, beta, out,
                      out_dtype, ldo, M, N, K, acc_dump, workspace, workspace_bytes, (hipStream_t)stream);
}

extern "C" int llmq_gemm_fp8_quantized_output(const uint8_t* A, int a_format, int64_t lda, const uint8_t* B, int64_t ldb,
                                              const float* a_scale, const float* w_scale, float alpha,
                                              const float* alpha_dev, const void* bias, int bias_dtype, float beta,
                                              const float* out_scale, float* out, int inter_dtype, int64_t ldo, int64_t M,
                                              int64_t N, int64_t K, void* workspace, size_t workspace_bytes,
                                              llmq_stream_t stream) {
    if (!out_scale) return LLMQ_ERR_NULL;
    // the few-token kernel is not used here: size the workspace for the tile kernel's plan
    return gemm_entry(1, a_format, A, lda, B, ldb, a_scale, w_scale, alpha, alpha_dev, bias, bias_dtype, beta, out,
                      inter_dtype, ldo, M, N, K, nullptr, workspace, workspace_bytes, (hipStream_t)stream, out_scale);
}

extern "C" size_t llmq_gemm_fp8_quantized_output_workspace_bytes(int64_t M, int64_t N, int64_t K) {
    if (M <= 0 || N <= 0 || K <= 0) return 0;
    const Plan p = make_plan(M, N, K, 1.0, true);
    return p.splits > 1 ? (size_t)p.splits * M * N * 4 : 0;
}

extern "C" size_t llmq_gemm_f16_workspace_bytes(int64_t M, int64_t N, int64_t K) {
    if (M <= 0 || N <= 0 || K <= 0) return 0;
    const Plan p = make_plan(M, N, 2 * K, 2.0);
    return p.splits > 1 ? (size_t)p.splits * M * N * 4 : 0;
}

extern "C" int llmq_gemm_f16(const void* A, int64_t lda, const void* B, int64_t ldb, float alpha, const void* bias,
                             int bias_dtype, float beta, void* out, int out_dtype, int64_t ldo, int64_t M, int64_t N,
                             int64_t K, float* acc_dump, void* workspace, size_t workspace_bytes, llmq_stream_t stream) {
    if (K < 0 || (K & 7) || (lda & 7) || (ldb & 7)) return LLMQ_ERR_SHAPE;  // 16-byte pieces of fp16
    return gemm_entry(2, 0, (const uint8_t*)A, 2 * lda, (const uint8_t*)B, 2 * ldb, nullptr, nullptr, alpha, nullptr, bias,
                      bias_dtype, beta, out, out_dtype, ldo, M, N, 2 * K, acc_dump, workspace, workspace_bytes,
                      (hipStream_t)stream);
}
