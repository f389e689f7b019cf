// Tile GEMM kernels for e4m3 x e4m3 -> fp32: every tile configuration of gemm_tile_impl.h instantiated for this operand format.
#include "gemm_tile_impl.h"

namespace llmq {

int launch_gemm_fp8_e4m3(LLMQ_GEMM_LAUNCH_ARGS) {
    return launch_gemm<true, 0>(A, lda, B, ldb, M, N, K, p, ep, out, ldo, acc_dump, ws, allow_dma, st);
}

}  // namespace llmq
