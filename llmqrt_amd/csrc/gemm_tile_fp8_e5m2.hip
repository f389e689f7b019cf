// Tile GEMM kernels for e5m2 x e4m3 -> fp32: every tile configuration of gemm_tile_impl.h instantiated for this operand format.
#include "gemm_tile_impl.h"

namespace llmq {

int launch_gemm_fp8_e5m2(LLMQ_GEMM_LAUNCH_ARGS) {
    return launch_gemm<true, 1>(A, lda, B, ldb, M, N, K, p, ep, out, ldo, acc_dump, ws, allow_dma, st);
}

}  // namespace llmq
