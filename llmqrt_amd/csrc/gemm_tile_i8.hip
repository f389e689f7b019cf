// Tile GEMM kernels for int8 x int8 -> int32: every tile configuration of gemm_tile_impl.h instantiated for this operand format.
#include "gemm_tile_impl.h"

namespace llmq {

int launch_gemm_i8(LLMQ_GEMM_LAUNCH_ARGS) {
    return launch_gemm<false, 0>(A, lda, B, ldb, M, N, K, p, ep, out, ldo, acc_dump, ws, allow_dma, st);
}

}  // namespace llmq
