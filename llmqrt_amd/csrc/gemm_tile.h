// Tile GEMM (int8 / fp8 / fp16 on the gfx950 matrix cores): the types and entry points shared by the planner
// (gemm_mfma.hip) and the translation units that instantiate the kernels for one operand format each
// (gemm_tile_i8.hip, gemm_tile_fp8.hip, gemm_tile_fp8_e5m2.hip, gemm_tile_f16.hip), so that they compile in parallel.
#pragma once
#include <cstddef>
#include <cstdint>

#include <hip/hip_runtime.h>

namespace llmq {

struct Epilogue {
    const float* a_scale;   // [M] or null
    const float* w_scale;   // [N] or null
    const float* alpha_dev; // device scalar or null
    const void* bias;       // [N] or null
    float alpha, beta;
    int bias_dtype, out_dtype;
    const float* out_scale;  // device scalar or null.  Set: the value rounded to out_dtype makes a round trip through
                             // e4m3fn on this scale and `out` is fp32 [M, N] (FP8 static linear with quantize_output)
};

struct Plan {
    int cfg;     // index into the config table
    int splits;  // K splits (1 = fused epilogue)
    int k_per_split;
};

constexpr int kNumCu = 256;
inline int cdiv(int64_t a, int64_t b) { return (int)((a + b - 1) / b); }
struct TileShape { int bm, bn, bk; };
constexpr TileShape kShapes[] = {
    {256, 256, 64},   // 0: 4 waves x (128x128)
    {256, 256, 64},   // 1: 8 waves x (128x64)
    {256, 128, 64},   // 2: 4 waves x (128x64)
    {128, 128, 64},   // 3: 4 waves x (64x64)
    {64, 128, 128},   // 4: 4 waves x (32x64)
    {32, 128, 128},   // 5: 4 waves x (32x32), decode
    {256, 256, 128},  // 6: 8 waves x (128x64), whole 128-byte lines per row (fp8 prefill)
    {128, 256, 128},  // 7: 8 waves x (64x64): twice the tiles of config 6 for grids that would leave CUs idle
};
constexpr int kNumShapes = sizeof(kShapes) / sizeof(kShapes[0]);

// One launch of the tile kernel (plus the reduction kernel of a K split) for the plan's tile configuration.
// allow_dma = false keeps the register-staged main loop (a ragged K tail always does).
#define LLMQ_GEMM_LAUNCH_ARGS                                                                                   \
    const uint8_t *A, int64_t lda, const uint8_t *B, int64_t ldb, int M, int N, int K, const Plan &p,            \
        const Epilogue &ep, void *out, int64_t ldo, void *acc_dump, void *ws, bool allow_dma, hipStream_t st
int launch_gemm_i8(LLMQ_GEMM_LAUNCH_ARGS);
int launch_gemm_f16(LLMQ_GEMM_LAUNCH_ARGS);       // K, lda, ldb in bytes
int launch_gemm_fp8_e4m3(LLMQ_GEMM_LAUNCH_ARGS);  // A in e4m3
int launch_gemm_fp8_e5m2(LLMQ_GEMM_LAUNCH_ARGS);  // A in e5m2, B in e4m3

}  // namespace llmq
