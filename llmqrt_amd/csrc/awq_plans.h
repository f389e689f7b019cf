// Launch plans of the AWQ kernels that live in their own translation units (awq_tile.hip, awq_decode.hip) and are
// dispatched from awq.hip.  One definition of each struct for all three files.
#pragma once
#include <cstddef>
#include <cstdint>

#include <hip/hip_runtime.h>

namespace llmq {

// Tile kernel for many tokens (awq_tile.hip).
// Tile shapes: 0 = 64 tokens x 128 channels (4 wavefronts), 1 = 256 x 256 (8 wavefronts), 2 = 128 x 128 (4 wavefronts).
struct AwqTilePlan { int cfg, splits, k_per_split; };
AwqTilePlan make_awq_tile_plan(int64_t M, int64_t N, int64_t K, int force_cfg, int force_splits);
void set_awq_tile_direct_loads(int on);  // 0: register-staged activation loads only
int launch_awq_tile(const AwqTilePlan& p, const uint16_t* x, int64_t ldx, const uint32_t* qw, const uint16_t* scales,
                    const uint32_t* qz, const uint16_t* bias, uint16_t* out, float* ws, int M, int N, int K, int G,
                    hipStream_t st);

// Decode kernel for up to 16 tokens (awq_decode.hip): cs wavefronts per column tile, pd stages ahead, ks K slices
// inside a block, splits blocks along K with groups_per_block groups each.
struct AwqDecodePlan { int cs, pd, splits, groups_per_block, ks; };
// The first kAwqTicketBytes of an AWQ workspace hold the arrival counters of the few-token kernel's K split: zero
// between calls (the caller clears them once, llmq_awq_workspace_init); the partial sums of every kernel follow.
constexpr size_t kAwqTicketBytes = (size_t)512 << 10;
int awq_clear_tickets(void* workspace, size_t bytes, hipStream_t st);
bool awq_decode_supported(int64_t M, int64_t N, int64_t K, int64_t group);
AwqDecodePlan make_awq_decode_plan(int64_t M, int64_t N, int64_t K, int force_cs, int force_pd, int force_splits, int force_ks);
size_t awq_decode_workspace_bytes(const AwqDecodePlan& p, int64_t M, int64_t N);
int launch_awq_decode(const AwqDecodePlan& p, const uint16_t* x, int64_t ldx, const uint32_t* qw, const uint16_t* scales,
                      const uint32_t* qz, const uint16_t* bias, uint16_t* out, unsigned int* tickets, float* ws, int M,
                      int N, int K, hipStream_t st);

}  // namespace llmq
