// Tile GEMM kernels for fp16 x fp16 -> fp32: every tile configuration of gemm_tile_impl.h instantiated for this operand format.
#include "gemm_tile_impl.h"

namespace llmq {

int launch_gemm_f16(LLMQ_GEMM_LAUNCH_ARGS) {
    return launch_gemm<false, 2>(A, lda, B, ldb, M, N, K, p, ep, out, ldo, acc_dump, ws, allow_dma, st);
}

}  // namespace llmq
