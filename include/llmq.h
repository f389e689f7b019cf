/* llmq.h - C ABI of libllmq_gfx950.so: the quantized-linear hot path of LLMQRT as
 * hand-written HIP kernels for AMD Instinct MI355X (gfx950 / CDNA4).
 *
 * Conventions
 *  - Every pointer is a DEVICE pointer unless its comment says "host".
 *  - The caller owns every buffer (inputs, outputs, workspaces); the library allocates
 *    nothing, never synchronises with the host and launches on the stream it is given
 *    (0 = the null stream).  Calls are asynchronous.  State kept between calls: the
 *    *_force_plan tuning hooks, and a 1 MiB ring of arrival counters per GPU (a static device
 *    array) for the K split of the few-token AWQ kernel, which ends inside one launch.  The
 *    counters are zero between calls and every call takes fresh slots, so calls on different
 *    streams do not share any; a captured call replays on the slots it was captured with, so
 *    two replays of one graph must not run concurrently.
 *  - Matrices are row-major; `ld*` is the row stride in ELEMENTS.
 *  - Return value: LLMQ_OK (0) or a negative llmq_status; llmq_status_string() names it.
 *  - Paths below are relative to the reference's runtime/ directory.
 */
#ifndef LLMQ_H_
#define LLMQ_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void* llmq_stream_t; /* a hipStream_t */

typedef enum {
    LLMQ_OK = 0,
    LLMQ_ERR_NULL = -1,      /* a required pointer is NULL */
    LLMQ_ERR_DTYPE = -2,     /* unsupported dtype / format selector */
    LLMQ_ERR_SHAPE = -3,     /* negative size, stride smaller than the row, unsupported alignment */
    LLMQ_ERR_WORKSPACE = -4, /* workspace missing or too small */
    LLMQ_ERR_LAUNCH = -5,    /* the HIP runtime refused the launch (hipGetLastError) */
    LLMQ_ERR_ALIGN = -6,     /* a pointer is not 16-byte aligned */
    LLMQ_ERR_SCRATCH = -7    /* the problem needs more scratch than the library's static array holds */
} llmq_status;

typedef enum { LLMQ_BF16 = 0, LLMQ_F16 = 1, LLMQ_F32 = 2 } llmq_dtype;
typedef enum { LLMQ_E4M3 = 0, LLMQ_E5M2 = 1 } llmq_fp8_format; /* OCP e4m3fn / e5m2 */

int llmq_abi_version(void);
const char* llmq_status_string(int status); /* host pointer to a static string */

/* ------------------------------------------------------------------------------------
 * Activation quantizers.  The reference runs each of these as 5-7 eager torch ops.
 * All arithmetic follows the reference bit for bit: it is carried out in the dtype of x
 * (the clamp bound, the scale and the quotient x/scale are each rounded to x_dtype).
 * x: [M, K] bf16/f16, K % 8 == 0, ldx % 8 == 0, 16-byte aligned.
 * ------------------------------------------------------------------------------------ */

/* Replaces quantize_activation_per_token_absmax, nn_models/modules/linear/linear_sq.py:55-65.
 * q: int8 [M, K] contiguous.  scale: [M] in x_dtype (scale_dtype == x_dtype) or fp32
 * (scale_dtype == LLMQ_F32, the same value widened - what the GEMM epilogue consumes). */
int llmq_quant_i8_per_token(const void* x, int x_dtype, int64_t M, int64_t K, int64_t ldx,
                            int8_t* q, void* scale, int scale_dtype, llmq_stream_t stream);

/* Replaces quantize_activation_per_tensor_absmax, linear_sq.py:44-53.  scale: one element.
 * workspace: >= llmq_quant_workspace_bytes() bytes, contents irrelevant on entry. */
int llmq_quant_i8_per_tensor(const void* x, int x_dtype, int64_t M, int64_t K, int64_t ldx,
                             int8_t* q, void* scale, int scale_dtype,
                             void* workspace, size_t workspace_bytes, llmq_stream_t stream);

/* The same two quantizers with the lower clamp bound of the absmax given by the caller instead of 1e-5:
 * absmax_floor = 1e-8 replaces dynamic_quantize_activation_per_token_absmax and
 * dynamic_quantize_activation_per_tensor_absmax, utils/quantization_utils.py:57-71 (which also overwrite
 * their input with the rounded quotients; x is left untouched here).  The bound is rounded to x_dtype
 * like every other value of the chain (1e-8 is 0 in fp16).  absmax_floor >= 0. */
int llmq_quant_i8_per_token_floor(const void* x, int x_dtype, int64_t M, int64_t K, int64_t ldx,
                                  int8_t* q, void* scale, int scale_dtype, float absmax_floor,
                                  llmq_stream_t stream);
int llmq_quant_i8_per_tensor_floor(const void* x, int x_dtype, int64_t M, int64_t K, int64_t ldx,
                                   int8_t* q, void* scale, int scale_dtype, float absmax_floor,
                                   void* workspace, size_t workspace_bytes, llmq_stream_t stream);

/* Replaces per_token_quantize, nn_models/modules/linear/linear_fp8.py:40-63.
 * q: e4m3fn bytes [M, K] contiguous; scale: fp32 [M]. */
int llmq_quant_fp8_per_token(const void* x, int x_dtype, int64_t M, int64_t K, int64_t ldx,
                             uint8_t* q, float* scale, llmq_stream_t stream);

/* Replaces per_tensor_quantize, linear_fp8.py:11-32.  scale: fp32, one element. */
int llmq_quant_fp8_per_tensor(const void* x, int x_dtype, int64_t M, int64_t K, int64_t ldx,
                              uint8_t* q, float* scale,
                              void* workspace, size_t workspace_bytes, llmq_stream_t stream);

/* Replaces static_per_tensor_quantize, linear_fp8.py:34-37.  scale: fp32 device scalar; the
 * quotient x / scale is kept in fp32 (torch: tensor / fp32 tensor promotes) when
 * scale_is_f32_tensor != 0, else it is rounded to x_dtype (torch: tensor / Python float). */
int llmq_quant_fp8_static(const void* x, int x_dtype, int64_t M, int64_t K, int64_t ldx,
                          uint8_t* q, const float* scale, int scale_is_f32_tensor,
                          llmq_stream_t stream);

/* Replaces quantize_weight_per_channel_absmax, utils/quantization_utils.py:27-38 (the offline weight
 * quantizer behind SqW8A8BBF16OBF16PerChannel.from_float).  w: [N, K] bf16 / f16 / f32, row stride ldw, any K;
 * q: int8 [N, K] contiguous; scale: [N] in w_dtype = absmax / 127 without a floor (an all-zero row quantizes
 * to zeros with a NaN scale, as in the reference).  Arithmetic in w_dtype, as the reference's tensor ops on the GPU. */
int llmq_quant_i8_weight_per_channel(const void* w, int w_dtype, int64_t N, int64_t K, int64_t ldw,
                                     int8_t* q, void* scale, llmq_stream_t stream);

size_t llmq_quant_workspace_bytes(void);

/* ------------------------------------------------------------------------------------
 * RMSNorm, alone or fused with the per-token quantizer of the Linear that follows it.
 * Replaces RMSNorm.forward (nn_models/modules/nonlinear/norm.py:10-16), and for the fused
 * forms also the quantizer call of the next Linear (block.py:68,76 -> linear_sq.py:55-65 /
 * linear_fp8.py:40-63): the activations make one trip through HBM instead of three.
 *   h = fp32(x); inv = 1/sqrt(mean_k(h^2) + eps); n = x_dtype(h * inv); y = x_dtype(weight * n)
 * x: [M, K] bf16/f16 (K % 8 == 0, ldx % 8 == 0, 16-byte aligned); weight: [K] in x_dtype.
 * y: [M, K] contiguous in x_dtype - required by llmq_rmsnorm, optional (may be NULL) for the
 * fused forms, which then never write the normalised activations.  q / scale: as for
 * llmq_quant_i8_per_token / llmq_quant_fp8_per_token applied to y.  inv_rms: optional fp32
 * [M] that receives inv (parity checks).  Given inv, every output is bit-identical to the
 * reference; inv itself depends on the summation order of the mean.
 * ------------------------------------------------------------------------------------ */
int llmq_rmsnorm(const void* x, int x_dtype, int64_t M, int64_t K, int64_t ldx,
                 const void* weight, float eps, void* y, float* inv_rms, llmq_stream_t stream);
int llmq_rmsnorm_quant_i8_per_token(const void* x, int x_dtype, int64_t M, int64_t K, int64_t ldx,
                                    const void* weight, float eps, void* y,
                                    int8_t* q, void* scale, int scale_dtype,
                                    float* inv_rms, llmq_stream_t stream);
int llmq_rmsnorm_quant_fp8_per_token(const void* x, int x_dtype, int64_t M, int64_t K, int64_t ldx,
                                     const void* weight, float eps, void* y,
                                     uint8_t* q, float* scale,
                                     float* inv_rms, llmq_stream_t stream);

/* ------------------------------------------------------------------------------------
 * W8A8 int8 GEMM.  Replaces w8a8_int8_linear_bbf16_obf16_per_tensor
 * (csrc/smoothquant/sq_gemm.cu:36-160, bound at csrc/bindings.cpp:10-11) and implements the
 * per-token x per-channel op the reference only declares
 * (w8a8_int8_linear_bbf16_obf16_per_channel, csrc/smoothquant/sq_gemm.h:19-24).
 *
 *   acc[m,n] = sum_k A[m,k] * B[n,k]                         (int32, exact)
 *   out[m,n] = out_dtype( f(acc[m,n]) )
 *     a_scale == NULL && w_scale == NULL:  f = alpha' * acc + beta * bias[n]
 *     otherwise:                           f = (acc * sa[m]) * sw[n] * alpha' + beta * bias[n]
 *   alpha' = alpha * (alpha_dev ? *alpha_dev : 1); sa/sw default to 1 when NULL; bias may be NULL.
 *
 * A: int8 [M,K] (lda >= K).  B: int8 [N,K] row-major (ldb >= K) - the reference passes the
 * same memory as a [K,N] view with stride (1,K).  K % 16 == 0, lda % 16 == 0, ldb % 16 == 0.
 * a_scale: fp32 [M]; w_scale: fp32 [N]; alpha_dev: fp32 device scalar (removes the
 * reference's .item() host syncs, linear_sq.py:127); bias: [N] of bias_dtype (bf16/f16/f32).
 * out: [M,N] bf16/f16 (ldo >= N).  acc_dump: optional int32 [M,N] contiguous that receives
 * the raw accumulators (parity checks).  workspace: >= llmq_gemm_workspace_bytes(M,N,K)
 * bytes (may be NULL when that is 0); contents irrelevant on entry.
 * ------------------------------------------------------------------------------------ */
int llmq_gemm_w8a8(const int8_t* A, int64_t lda, const int8_t* B, int64_t ldb,
                   const float* a_scale, const float* w_scale,
                   float alpha, const float* alpha_dev,
                   const void* bias, int bias_dtype, float beta,
                   void* out, int out_dtype, int64_t ldo,
                   int64_t M, int64_t N, int64_t K,
                   int32_t* acc_dump, void* workspace, size_t workspace_bytes,
                   llmq_stream_t stream);

/* ------------------------------------------------------------------------------------
 * FP8 scaled GEMM.  Replaces f8f8bf16_rowwise (csrc/fp8/sm89_fp8_rowwise_fbgemm.cu:582-606,
 * bound as cutlass_f8f8bf16_rowwise_sm89 at csrc/bindings.cpp:13) and f8f8bf16_tensorwise
 * (csrc/fp8/sm89_fp8_tensorwise_cutlassgemm.cu:316-334, bound at csrc/bindings.cpp:12).
 * Same contract as llmq_gemm_w8a8 with fp32 accumulation of exact fp8 products:
 * A: fp8 bytes [M,K] in a_format (e4m3fn or e5m2); B: e4m3fn bytes [N,K].
 * acc_dump: optional fp32 [M,N].
 * ------------------------------------------------------------------------------------ */
int llmq_gemm_fp8(const uint8_t* A, int a_format, int64_t lda, const uint8_t* B, int64_t ldb,
                  const float* a_scale, const float* w_scale,
                  float alpha, const float* alpha_dev,
                  const void* bias, int bias_dtype, float beta,
                  void* out, int out_dtype, int64_t ldo,
                  int64_t M, int64_t N, int64_t K,
                  float* acc_dump, void* workspace, size_t workspace_bytes,
                  llmq_stream_t stream);

size_t llmq_gemm_workspace_bytes(int64_t M, int64_t N, int64_t K);

/* llmq_gemm_fp8 with the output quantization of FP8StaticLinear.forward folded into the epilogue
 * (nn_models/modules/linear/linear_fp8.py:309-311: static_per_tensor_quantize(output, output_scale), then
 * qoutput.to(dtype) * output_scale): the GEMM result is rounded to inter_dtype (bf16 / f16, the module's dtype),
 * divided by *out_scale in fp32, clamped to +-448, rounded to e4m3fn, widened again and multiplied by *out_scale.
 * out: fp32 [M, N] (the reference's product of a 16-bit tensor and a one-element fp32 tensor is fp32), row stride
 * ldo elements.  out_scale: fp32 device scalar.  One launch instead of three and no extra trips of the [M, N] output
 * through HBM.  workspace: >= llmq_gemm_fp8_quantized_output_workspace_bytes(M, N, K). */
int llmq_gemm_fp8_quantized_output(const uint8_t* A, int a_format, int64_t lda, const uint8_t* B, int64_t ldb,
                                   const float* a_scale, const float* w_scale,
                                   float alpha, const float* alpha_dev,
                                   const void* bias, int bias_dtype, float beta,
                                   const float* out_scale, float* out, int inter_dtype, int64_t ldo,
                                   int64_t M, int64_t N, int64_t K,
                                   void* workspace, size_t workspace_bytes, llmq_stream_t stream);
size_t llmq_gemm_fp8_quantized_output_workspace_bytes(int64_t M, int64_t N, int64_t K);

/* llmq_gemm_w8a8 for callers that cannot allocate or pass a workspace: code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc.  No counterpart in the reference.  Same arguments and
 * results as llmq_gemm_w8a8 without acc_dump / workspace: the split-K partial sums go to a static device array
 * of llmq_gemm_static_scratch_bytes() (32 MiB) that every GPU holds from library load to process exit.  The
 * call allocates nothing (no hipMalloc / hipFree), looks the array's device address up once per device (on the
 * first call there: make that call outside a graph capture).  Arguments are validated as in llmq_gemm_w8a8; then
 * LLMQ_ERR_SCRATCH is returned, before any launch, when the partial sums of the K split planned for this int8
 * problem (splits x M x N x 4 bytes; llmq_gemm_workspace_bytes(M, N, K) is an upper bound) exceed the array.  All calls on one GPU share the array: two calls that
 * overlap in time (different streams) race; calls on one stream are ordered and safe.  Nothing in the array has
 * to start at zero: every partial sum is written before it is read. */
int llmq_gemm_w8a8_static(const int8_t* A, int64_t lda, const int8_t* B, int64_t ldb,
                          const float* a_scale, const float* w_scale,
                          float alpha, const float* alpha_dev,
                          const void* bias, int bias_dtype, float beta,
                          void* out, int out_dtype, int64_t ldo,
                          int64_t M, int64_t N, int64_t K, llmq_stream_t stream);
size_t llmq_gemm_static_scratch_bytes(void);

/* fp16 GEMM with fp32 accumulation, out = alpha * A B^T + beta * bias: replaces the torch.matmul of the reference's
 * many-token AWQ path (nn_models/modules/linear/linear_awq.py:51-53) after llmq_awq_dequant_t.  A: fp16 [M, K], B: fp16
 * [N, K] (both K-contiguous, K % 8 == 0, lda % 8 == 0, ldb % 8 == 0, 16-byte aligned); bias: [N] or null; out: bf16 / f16
 * [M, N].  Same tile kernels, plans and workspace rule as llmq_gemm_w8a8 (llmq_gemm_f16_workspace_bytes). */
int llmq_gemm_f16(const void* A, int64_t lda, const void* B, int64_t ldb, float alpha, const void* bias, int bias_dtype,
                  float beta, void* out, int out_dtype, int64_t ldo, int64_t M, int64_t N, int64_t K, float* acc_dump,
                  void* workspace, size_t workspace_bytes, llmq_stream_t stream);
size_t llmq_gemm_f16_workspace_bytes(int64_t M, int64_t N, int64_t K);

/* Few-token quantized linear in ONE launch: per-token dynamic activation quantizer + GEMM + per-token x per-channel
 * epilogue, for M <= llmq_linear_dynamic_max_tokens(K) tokens (16, or fewer when 16 quantized rows of K + 16 bytes do not
 * fit in 64 KB of LDS: 3 at K = 18944).  Replaces the two steps of
 * SqW8A8BBF16OBF16PerChannel.forward / the per-token branch of FP8DynamicLinear.forward
 * (nn_models/modules/linear/linear_sq.py:97-138 with the quantizer of lines 55-65;
 * nn_models/modules/linear/linear_fp8.py:40-63 and 199-221) and gives, bit for bit, what
 * llmq_quant_i8_per_token (llmq_quant_fp8_per_token) followed by llmq_gemm_w8a8 (llmq_gemm_fp8) with a_scale = the
 * quantizer's scales, alpha = beta = 1 gives:
 *   out[m, n] = out_dtype( ((sum_k q[m, k] B[n, k]) * s[m]) * w_scale[n] + bias[n] ).
 * x: bf16 / f16 [M, K], row stride ldx (K % 16 == 0, ldx % 8 == 0); B: int8 / e4m3 [N, K], row stride ldb; w_scale: [N]
 * or null; bias: [N] or null; out: bf16 / f16 [M, N].  Optional outputs for checking: q_dump [M, K] (the codes),
 * scale_dump [M] (fp32), acc_dump [M, N] (raw accumulators).  No workspace.  More tokens return LLMQ_ERR_SHAPE. */
int llmq_linear_i8_dynamic(const void* x, int x_dtype, int64_t ldx, const int8_t* B, int64_t ldb, const float* w_scale,
                           const void* bias, int bias_dtype, void* out, int out_dtype, int64_t ldo, int64_t M, int64_t N,
                           int64_t K, int8_t* q_dump, float* scale_dump, int32_t* acc_dump, llmq_stream_t stream);
int llmq_linear_fp8_dynamic(const void* x, int x_dtype, int64_t ldx, const uint8_t* B, int64_t ldb, const float* w_scale,
                            const void* bias, int bias_dtype, void* out, int out_dtype, int64_t ldo, int64_t M, int64_t N,
                            int64_t K, uint8_t* q_dump, float* scale_dump, float* acc_dump, llmq_stream_t stream);
int llmq_linear_dynamic_max_tokens(int64_t K);
/* Tuning / test hook: 0 = two 16-channel tiles per wavefront x 4 wavefronts per block, 1 = one tile x 8 wavefronts,
 * -1 = built-in choice.  Per host thread (thread-local state): it affects only calls made later by the thread that set it. */
int llmq_linear_dynamic_force_variant(int v);

/* Tuning / test hook with no counterpart in the reference: force tile configuration `cfg`
 * (0 .. llmq_gemm_num_configs()-1) and K split `splits` for every later GEMM call of this
 * process; cfg < 0 restores the built-in heuristic.  cfg | 64 keeps the register-staged main loop,
 * 100 .. 105 pick a variant of the few-token kernel.  Per host thread (thread-local state): it affects only calls made later by the thread that set it. */
int llmq_gemm_force_plan(int cfg, int splits);
int llmq_gemm_num_configs(void);

/* ------------------------------------------------------------------------------------
 * AWQ W4A16.  Replaces awq_gemm_triton / awq_dequantize_triton
 * (triton_kernels/awq_kernels.py:328-378 / :273-320).
 * qweight: int32 [K, N/8], nibble i of a word = logical column 8c + {0,2,4,6,1,3,5,7}[i]
 * (nn_models/modules/linear/linear_awq.py:192-202); qzeros: int32 [K/G, N/8], same packing;
 * scales: fp16 [K/G, N].  G (group) divides K, G % 32 == 0; N % 8 == 0.
 * ------------------------------------------------------------------------------------ */

/* out[m,n] = fp16( sum_k x[m,k] * fp16((q[k,n] - z[k/G,n]) * s[k/G,n]) + bias[n] ), fp32
 * accumulation in a fixed order (deterministic, unlike the reference's fp16 atomics).
 * x: fp16 [M,K] (ldx >= K, K % 32 == 0); out: fp16 [M,N] contiguous; bias: fp16 [N] or NULL.
 * Up to 64 tokens a streaming kernel runs (for group 128 the weights enter the matrix core
 * unrounded, exact (q - z) * s in fp32, instead of rounded to fp16 first); above 64 tokens
 * an fp16 tile GEMM dequantizes the weights on their way into LDS.  All are within 1e-2 of the
 * dequantize-then-matmul math.
 * workspace: >= llmq_awq_gemm_workspace_bytes(M,N,K) bytes, 16-byte aligned.  Its first
 * llmq_awq_workspace_ticket_bytes() bytes are the arrival counters of the few-token kernel's K split:
 * they must be zero when a call starts and every call leaves them zero, so a workspace is cleared once
 * (llmq_awq_workspace_init, or any zero fill) when it is allocated and can then serve any sequence of calls
 * of any shape; the contents of the rest are irrelevant.  Calls that may overlap in time (different
 * streams, a captured launch replayed beside eager calls) need different workspaces. */
int llmq_awq_gemm(const void* x, int64_t ldx, const int32_t* qweight, const void* scales,
                  const int32_t* qzeros, const void* bias, void* out,
                  int64_t M, int64_t N, int64_t K, int64_t group,
                  void* workspace, size_t workspace_bytes, llmq_stream_t stream);

size_t llmq_awq_gemm_workspace_bytes(int64_t M, int64_t N, int64_t K);

/* No counterpart in the reference (its split-K ends in fp16 atomics on the output, awq_kernels.py:253-267):
 * size of the counter area at the start of an AWQ workspace, and a launch on `stream` that zeroes it. */
size_t llmq_awq_workspace_ticket_bytes(void);
int llmq_awq_workspace_init(void* workspace, size_t workspace_bytes, llmq_stream_t stream);

/* Tuning / test hook with no counterpart in the reference: force the kernel variant of
 * llmq_awq_gemm for every later call of this process: v = 1 or 2 words per lane of the streaming
 * kernel in 16-token slabs, 5 or 6 = streaming kernel with 2 or 4 token tiles per wavefront,
 * 3, 7 or 4 = tile kernel with 64x128, 128x128 or 256x256 tiles (any M), 8 .. 11 = the few-token kernel
 * (M <= 64; 128- / 256-byte row segments, one / two stages ahead), 0 = heuristic; the cross-block K split
 * (0 = heuristic); the wavefronts per block along K of the streaming kernel (4 or 8), or the K slices
 * inside a block of the few-token kernel (1, 2 or 4, v = 8 only); 0 = heuristic.
 * v + 32 keeps the tile kernel's register-staged activation loads (default: straight into LDS when K % 64 == 0).
 * Per host thread (thread-local state): it affects only calls made later by the thread that set it. */
int llmq_awq_force_plan(int v, int splits, int k_waves);

/* out: fp16 [K, N] contiguous = fp16(q - z) * s, bit-exact with
 * utils/packing_utils.py:65-80 (dequantize_gemm). */
int llmq_awq_dequant(const int32_t* qweight, const void* scales, const int32_t* qzeros,
                     void* out, int64_t K, int64_t N, int64_t group, llmq_stream_t stream);

/* The same dequantized weights written as the transpose, fp16 [N, K] with K contiguous (the B operand of
 * llmq_gemm_f16): together they replace awq_dequantize_triton + torch.matmul of the reference's many-token path
 * (nn_models/modules/linear/linear_awq.py:49-53).  group % 8 == 0. */
int llmq_awq_dequant_t(const int32_t* qweight, const void* scales, const int32_t* qzeros, void* out,
                       int64_t K, int64_t N, int64_t group, llmq_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* LLMQ_H_ */
