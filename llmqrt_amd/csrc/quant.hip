// Activation quantizers (int8 SmoothQuant and OCP e4m3fn FP8), one fused HIP kernel each.
//
// The reference runs these as chains of eager torch ops in the activation dtype
// (nn_models/modules/linear/linear_sq.py:44-65, nn_models/modules/linear/linear_fp8.py:11-63):
//   scale = round_dt( max(absmax, round_dt(floor)) / qmax )
//   q     = narrow( clamp( round_dt( x / scale ) ) )
// The kernels reproduce exactly that sequence of roundings.  They are HBM-bound:
// 2 bytes read + 1 byte written per element, one row per 256-thread block, the row held in
// registers between the absmax pass and the quantize pass so x is read from HBM once.
#include "llmq_common.h"
#include "quant_math.h"

namespace llmq {
namespace {

constexpr int kThreads = 256;
constexpr int kNW = kThreads / kWave;
constexpr int kMaxPartials = 1024;  // per-tensor absmax partials (one per stage-1 block)

enum { SCALE_ROW = 0, SCALE_TENSOR = 1, SCALE_STATIC = 2 };

// One block of NT threads per row.  NC > 0: the row's 16-byte chunks (8 elements) are kept in NC
// registers per thread between the two passes; NC == 0: rows of any length, second pass
// re-reads x (served by L2).
template <int DT, int MODE, int SCALE, int NC, int NT = kThreads>
__global__ __launch_bounds__(NT) void quant_rows_kernel(
    const uint16_t* __restrict__ x, int64_t ldx, int64_t K, uint8_t* __restrict__ q,
    void* __restrict__ scale_out, int scale_dtype, const float* __restrict__ aux, int n_aux,
    int static_f32, float floor) {
    __shared__ float smem[NT / kWave];
    const int64_t row = blockIdx.x;
    const int tid = threadIdx.x;
    const int nchunk = (int)(K >> 3);
    const uint4* xr = reinterpret_cast<const uint4*>(x + row * ldx);
    uint2* qr = reinterpret_cast<uint2*>(q + row * K);

    uint4 cache[NC > 0 ? NC : 1];
    float s;
    bool fin = false;  // block-uniform: the absmax behind the scale is finite, so no quotient can be NaN
    if (SCALE == SCALE_ROW) {
        float amax = 0.f;
        if (NC > 0) {
#pragma unroll
            for (int c = 0; c < NC; c++) {
                const int i = tid + c * NT;
                cache[c] = (i < nchunk) ? xr[i] : make_uint4(0, 0, 0, 0);
            }
#pragma unroll
            for (int c = 0; c < NC; c++) amax = max_nonneg(amax, absmax8(cache[c], DT == LLMQ_BF16));
        } else {
            for (int i = tid; i < nchunk; i += NT) amax = max_nonneg(amax, absmax8(xr[i], DT == LLMQ_BF16));
        }
        amax = block_max<NT / kWave>(amax, smem);
        s = scale_from_amax<DT, MODE>(amax, floor);
        fin = amax < __builtin_inff() && s > 0.f;  // (the fp8 floor rounds to 0 in fp16: an all-zero row has scale 0 and 0 / 0)
    } else if (SCALE == SCALE_TENSOR) {
        float amax = 0.f;
        for (int i = tid; i < n_aux; i += NT) amax = max_nonneg(amax, aux[i]);
        amax = block_max<NT / kWave>(amax, smem);
        s = scale_from_amax<DT, MODE>(amax, floor);
        fin = amax < __builtin_inff() && s > 0.f;  // (the fp8 floor rounds to 0 in fp16: an all-zero row has scale 0 and 0 / 0)
    } else {
        s = aux[0];
    }
    if (SCALE != SCALE_STATIC && tid == 0 && (SCALE == SCALE_ROW || row == 0)) {
        const int64_t o = SCALE == SCALE_ROW ? row : 0;
        if (scale_dtype == LLMQ_F32) ((float*)scale_out)[o] = s;
        else ((uint16_t*)scale_out)[o] = Lo<DT>::from_f32(s);
    }
    const float inv_s = 1.0f / s;
    constexpr bool F32Q = (SCALE == SCALE_STATIC);
    if (SCALE == SCALE_ROW && NC > 0) {
        if (fin) {
#pragma unroll
            for (int c = 0; c < NC; c++) {
                const int i = tid + c * NT;
                if (i < nchunk) qr[i] = quant8<DT, MODE, Q_DT, true>(cache[c], s, inv_s);
            }
        } else {
#pragma unroll
            for (int c = 0; c < NC; c++) {
                const int i = tid + c * NT;
                if (i < nchunk) qr[i] = quant8<DT, MODE, Q_DT>(cache[c], s, inv_s);
            }
        }
    } else if (F32Q) {
        if (static_f32) {
            for (int i = tid; i < nchunk; i += NT) qr[i] = quant8<DT, MODE, Q_DIV_F32>(xr[i], s, inv_s);
        } else {
            for (int i = tid; i < nchunk; i += NT) qr[i] = quant8<DT, MODE, Q_DIV_DT>(xr[i], s, inv_s);
        }
    } else if (fin) {
        for (int i = tid; i < nchunk; i += NT) qr[i] = quant8<DT, MODE, Q_DT, true>(xr[i], s, inv_s);
    } else {
        for (int i = tid; i < nchunk; i += NT) qr[i] = quant8<DT, MODE, Q_DT>(xr[i], s, inv_s);
    }
}

// One wavefront per row, for rows of at most 64 * NCW chunks: no block barrier, the reductions are wavefront
// butterflies, and the four rows of a block are independent, so four times as many rows are in flight per CU.
template <int DT, int MODE, int NCW>
__global__ __launch_bounds__(kThreads) void quant_rows_wave_kernel(
    const uint16_t* __restrict__ x, int64_t ldx, int64_t K, int64_t M, uint8_t* __restrict__ q,
    void* __restrict__ scale_out, int scale_dtype, float floor) {
    const int lane = threadIdx.x & (kWave - 1);
    const int64_t row = (int64_t)blockIdx.x * kNW + threadIdx.x / kWave;
    if (row >= M) return;  // wavefront-uniform; the kernel has no barrier
    const int nchunk = (int)(K >> 3);
    const uint4* xr = reinterpret_cast<const uint4*>(x + row * ldx);
    uint2* qr = reinterpret_cast<uint2*>(q + row * K);
    uint4 cache[NCW];
#pragma unroll
    for (int c = 0; c < NCW; c++) {
        const int i = lane + c * kWave;
        cache[c] = (i < nchunk) ? xr[i] : make_uint4(0, 0, 0, 0);
    }
    float amax = 0.f;
#pragma unroll
    for (int c = 0; c < NCW; c++) amax = max_nonneg(amax, absmax8(cache[c], DT == LLMQ_BF16));
    amax = wave_max(amax);
    const float s = scale_from_amax<DT, MODE>(amax, floor);
    if (lane == 0) {
        if (scale_dtype == LLMQ_F32) ((float*)scale_out)[row] = s;
        else ((uint16_t*)scale_out)[row] = Lo<DT>::from_f32(s);
    }
    const float inv_s = 1.0f / s;
    if (amax < __builtin_inff() && s > 0.f) {  // wavefront-uniform: no quotient can be NaN
#pragma unroll
        for (int c = 0; c < NCW; c++) {
            const int i = lane + c * kWave;
            if (i < nchunk) qr[i] = quant8<DT, MODE, Q_DT, true>(cache[c], s, inv_s);
        }
    } else {
#pragma unroll
        for (int c = 0; c < NCW; c++) {
            const int i = lane + c * kWave;
            if (i < nchunk) qr[i] = quant8<DT, MODE, Q_DT>(cache[c], s, inv_s);
        }
    }
}

// Stage 1 of the per-tensor quantizers: grid-stride absmax, one partial per block.
template <int DT>
__global__ __launch_bounds__(kThreads) void absmax_partials_kernel(
    const uint16_t* __restrict__ x, int64_t ldx, int64_t M, int64_t K, float* __restrict__ partials) {
    __shared__ float smem[kNW];
    const int64_t cpr = K >> 3, total = M * cpr;
    float amax = 0.f;
    for (int64_t i = (int64_t)blockIdx.x * kThreads + threadIdx.x; i < total; i += (int64_t)gridDim.x * kThreads) {
        const int64_t r = i / cpr, c = i - r * cpr;
        amax = max_nonneg(amax, absmax8(reinterpret_cast<const uint4*>(x + r * ldx)[c], DT == LLMQ_BF16));
    }
    amax = block_max<kNW>(amax, smem);
    if (threadIdx.x == 0) partials[blockIdx.x] = amax;
}

// ---- RMSNorm fused with the per-token quantizer --------------------------------------------
// The reference normalises (nn_models/modules/nonlinear/norm.py:10-16) and then quantizes the result in
// the first Linear of the block (nn_models/modules/nonlinear/block.py:68,76 -> linear_sq.py:55-65 /
// linear_fp8.py:40-63): two round trips of the activations through HBM.  Here a row is read once, kept
// in registers, normalised, (optionally) written back as y, and quantized:
//   h = fp32(x);  inv = 1 / sqrt(mean(h^2) + eps);  n = round_dt(h * inv);  y = round_dt(w * n)
//   then exactly the per-token quantizer above on y.
// Everything after `inv` is bit-identical to the reference evaluated with the same inv; inv itself
// depends on the summation order of mean() (here: per-thread FMA chain, wavefront butterfly, then the
// wavefronts in order) and can differ from another order in the last bits.
template <int DT>
__device__ __forceinline__ float sumsq8(uint4 r, float acc) {
    const uint32_t w[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const float a = Lo<DT>::to_f32((uint16_t)(w[i] & 0xffffu)), b = Lo<DT>::to_f32((uint16_t)(w[i] >> 16));
        acc = fmaf(a, a, acc);
        acc = fmaf(b, b, acc);
    }
    return acc;
}

template <int DT>
__device__ __forceinline__ uint4 norm8(uint4 r, uint4 wv, float inv) {
    const uint32_t x[4] = {r.x, r.y, r.z, r.w}, w[4] = {wv.x, wv.y, wv.z, wv.w};
    uint32_t o[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        // The reference rounds the product to fp32 and then to the activation dtype.  Keep the fp32 product
        // opaque so that the compiler cannot fuse multiply and narrowing into one mixed-precision
        // instruction, which rounds once and lands on the other side of a tie now and then.  The two narrowings of a
        // pair share one packed conversion.
        float p0 = Lo<DT>::lo_f32(x[i]) * inv;
        float p1 = Lo<DT>::hi_f32(x[i]) * inv;
        asm volatile("" : "+v"(p0), "+v"(p1));
        const uint32_t n = Lo<DT>::pack2(p0, p1);
        // (the product of two 16-bit floats is exact in fp32: narrowing it rounds once however it is compiled)
        o[i] = Lo<DT>::pack2(Lo<DT>::lo_f32(w[i]) * Lo<DT>::lo_f32(n), Lo<DT>::hi_f32(w[i]) * Lo<DT>::hi_f32(n));
    }
    return make_uint4(o[0], o[1], o[2], o[3]);
}

// QMODE: -1 = no quantizer (plain RMSNorm), MODE_I8, MODE_F8.
template <int DT, int QMODE, int NC, int NT = kThreads>
__global__ __launch_bounds__(NT) void rmsnorm_quant_rows_kernel(
    const uint16_t* __restrict__ x, int64_t ldx, int64_t K, const uint16_t* __restrict__ weight, float eps,
    uint16_t* __restrict__ y, uint8_t* __restrict__ q, void* __restrict__ scale_out, int scale_dtype,
    float* __restrict__ inv_out) {
    __shared__ float smem[NT / kWave];
    constexpr int QM = QMODE < 0 ? MODE_I8 : QMODE;
    const int64_t row = blockIdx.x;
    const int tid = threadIdx.x;
    const int nchunk = (int)(K >> 3);
    const uint4* xr = reinterpret_cast<const uint4*>(x + row * ldx);
    const uint4* wr = reinterpret_cast<const uint4*>(weight);
    uint4* yr = y ? reinterpret_cast<uint4*>(y + row * K) : nullptr;
    uint2* qr = reinterpret_cast<uint2*>(q + row * K);

    uint4 cache[NC > 0 ? NC : 1];
    float ss = 0.f;
    if (NC > 0) {
#pragma unroll
        for (int c = 0; c < NC; c++) {
            const int i = tid + c * NT;
            cache[c] = (i < nchunk) ? xr[i] : make_uint4(0, 0, 0, 0);
        }
#pragma unroll
        for (int c = 0; c < NC; c++) ss = sumsq8<DT>(cache[c], ss);
    } else {
        for (int i = tid; i < nchunk; i += NT) ss = sumsq8<DT>(xr[i], ss);
    }
    ss = block_sum<NT / kWave>(ss, smem);
    const float inv = 1.0f / sqrtf(ss / (float)K + eps);
    if (inv_out && tid == 0) inv_out[row] = inv;

    float amax = 0.f;
    if (NC > 0) {
#pragma unroll
        for (int c = 0; c < NC; c++) {
            const int i = tid + c * NT;
            if (i < nchunk) {
                cache[c] = norm8<DT>(cache[c], wr[i], inv);
                if (yr) yr[i] = cache[c];
                amax = max_nonneg(amax, absmax8(cache[c], DT == LLMQ_BF16));
            }
        }
    } else {
        for (int i = tid; i < nchunk; i += NT) {
            const uint4 v = norm8<DT>(xr[i], wr[i], inv);
            if (yr) yr[i] = v;
            amax = max_nonneg(amax, absmax8(v, DT == LLMQ_BF16));
        }
    }
    if (QMODE < 0) return;
    amax = block_max<NT / kWave>(amax, smem);
    const float s = scale_from_amax<DT, QM>(amax);
    if (tid == 0) {
        if (scale_dtype == LLMQ_F32) ((float*)scale_out)[row] = s;
        else ((uint16_t*)scale_out)[row] = Lo<DT>::from_f32(s);
    }
    const float inv_s = 1.0f / s;
    if (NC > 0 && amax < __builtin_inff() && s > 0.f) {  // block-uniform: no quotient can be NaN
#pragma unroll
        for (int c = 0; c < NC; c++) {
            const int i = tid + c * NT;
            if (i < nchunk) qr[i] = quant8<DT, QM, Q_DT, true>(cache[c], s, inv_s);
        }
    } else if (NC > 0) {
#pragma unroll
        for (int c = 0; c < NC; c++) {
            const int i = tid + c * NT;
            if (i < nchunk) qr[i] = quant8<DT, QM, Q_DT>(cache[c], s, inv_s);
        }
    } else {
        for (int i = tid; i < nchunk; i += NT) qr[i] = quant8<DT, QM, Q_DT>(norm8<DT>(xr[i], wr[i], inv), s, inv_s);
    }
}

// The same with one wavefront per row (see quant_rows_wave_kernel); the sum of squares is a per-lane FMA chain and a
// wavefront butterfly.
template <int DT, int QMODE, int NCW>
__global__ __launch_bounds__(kThreads) void rmsnorm_quant_rows_wave_kernel(
    const uint16_t* __restrict__ x, int64_t ldx, int64_t K, int64_t M, const uint16_t* __restrict__ weight, float eps,
    uint16_t* __restrict__ y, uint8_t* __restrict__ q, void* __restrict__ scale_out, int scale_dtype,
    float* __restrict__ inv_out) {
    constexpr int QM = QMODE < 0 ? MODE_I8 : QMODE;
    const int lane = threadIdx.x & (kWave - 1);
    const int64_t row = (int64_t)blockIdx.x * kNW + threadIdx.x / kWave;
    if (row >= M) return;  // wavefront-uniform; the kernel has no barrier
    const int nchunk = (int)(K >> 3);
    const uint4* xr = reinterpret_cast<const uint4*>(x + row * ldx);
    const uint4* wr = reinterpret_cast<const uint4*>(weight);
    uint4* yr = y ? reinterpret_cast<uint4*>(y + row * K) : nullptr;
    uint2* qr = reinterpret_cast<uint2*>(q + row * K);
    uint4 cache[NCW];
#pragma unroll
    for (int c = 0; c < NCW; c++) {
        const int i = lane + c * kWave;
        cache[c] = (i < nchunk) ? xr[i] : make_uint4(0, 0, 0, 0);
    }
    float ss = 0.f;
#pragma unroll
    for (int c = 0; c < NCW; c++) ss = sumsq8<DT>(cache[c], ss);
    ss = wave_sum(ss);
    const float inv = 1.0f / sqrtf(ss / (float)K + eps);
    if (inv_out && lane == 0) inv_out[row] = inv;
    float amax = 0.f;
#pragma unroll
    for (int c = 0; c < NCW; c++) {
        const int i = lane + c * kWave;
        if (i < nchunk) {
            cache[c] = norm8<DT>(cache[c], wr[i], inv);
            if (yr) yr[i] = cache[c];
            amax = max_nonneg(amax, absmax8(cache[c], DT == LLMQ_BF16));
        }
    }
    if (QMODE < 0) return;
    amax = wave_max(amax);
    const float s = scale_from_amax<DT, QM>(amax);
    if (lane == 0) {
        if (scale_dtype == LLMQ_F32) ((float*)scale_out)[row] = s;
        else ((uint16_t*)scale_out)[row] = Lo<DT>::from_f32(s);
    }
    const float inv_s = 1.0f / s;
    if (amax < __builtin_inff() && s > 0.f) {  // wavefront-uniform: no quotient can be NaN
#pragma unroll
        for (int c = 0; c < NCW; c++) {
            const int i = lane + c * kWave;
            if (i < nchunk) qr[i] = quant8<DT, QM, Q_DT, true>(cache[c], s, inv_s);
        }
    } else {
#pragma unroll
        for (int c = 0; c < NCW; c++) {
            const int i = lane + c * kWave;
            if (i < nchunk) qr[i] = quant8<DT, QM, Q_DT>(cache[c], s, inv_s);
        }
    }
}

// Measured with the inputs streamed from HBM: at K = 1024 and 8192 rows the wavefront-per-row kernels take 7.1 us
// (quantizer) / 9.7 us (RMSNorm + quantizer) against 9.3 / 13.7 us for a block per row; at K = 3584 a block per row is
// ahead by 5 % (17.2 against 18.0 us) and by 1.3 us at a few rows, so longer rows keep it.
inline bool wave_rows(int64_t M, int64_t K) { return (K >> 3) <= 2 * kWave && M >= 256; }
// Rows of 257-512 chunks (K = 3584: 448) with enough rows to fill the chip run on half-size blocks with four chunks
// per thread: the per-row arithmetic that every wavefront repeats (two reductions, the scale, its reciprocal) is spread
// over twice the elements.  Fused RMSNorm + int8 quantizer at 8192 x 3584 from HBM: 21.6 us against 23.6.
inline bool half_blocks(int64_t M, int64_t K) { return (K >> 3) > kThreads && (K >> 3) <= 2 * kThreads && M >= 256; }

template <int DT, int QMODE>
int launch_norm(const void* x, int64_t M, int64_t K, int64_t ldx, const void* weight, float eps, void* y, void* q,
                void* scale, int scale_dtype, float* inv_out, hipStream_t st) {
    const dim3 grid((unsigned)M), block(kThreads);
    const int64_t per_thread = ((K >> 3) + kThreads - 1) / kThreads;
    if (wave_rows(M, K)) {
        const dim3 wgrid((unsigned)((M + kNW - 1) / kNW));
        const int64_t per_lane = ((K >> 3) + kWave - 1) / kWave;
#define LLMQ_LAUNCH_NCW(NCW)                                                                                          \
    hipLaunchKernelGGL((rmsnorm_quant_rows_wave_kernel<DT, QMODE, NCW>), wgrid, block, 0, st, (const uint16_t*)x, ldx, K, \
                       M, (const uint16_t*)weight, eps, (uint16_t*)y, (uint8_t*)q, scale, scale_dtype, inv_out)
        if (per_lane <= 1) LLMQ_LAUNCH_NCW(1);
        else LLMQ_LAUNCH_NCW(2);
#undef LLMQ_LAUNCH_NCW
        return launch_status();
    }
#define LLMQ_LAUNCH_NCT(NC, NT)                                                                                          \
    hipLaunchKernelGGL((rmsnorm_quant_rows_kernel<DT, QMODE, NC, NT>), grid, dim3(NT), 0, st, (const uint16_t*)x, ldx, K, \
                       (const uint16_t*)weight, eps, (uint16_t*)y, (uint8_t*)q, scale, scale_dtype, inv_out)
#define LLMQ_LAUNCH_NC(NC) LLMQ_LAUNCH_NCT(NC, kThreads)
    if (half_blocks(M, K)) LLMQ_LAUNCH_NCT(4, kThreads / 2);
    else if (per_thread <= 1) LLMQ_LAUNCH_NC(1);
    else if (per_thread <= 2) LLMQ_LAUNCH_NC(2);
    else if (per_thread <= 4) LLMQ_LAUNCH_NC(4);
    else if (per_thread <= 10) LLMQ_LAUNCH_NC(10);
    else LLMQ_LAUNCH_NC(0);
#undef LLMQ_LAUNCH_NC
#undef LLMQ_LAUNCH_NCT
    return launch_status();
}

template <int QMODE>
int rmsnorm_entry(const void* x, int x_dtype, int64_t M, int64_t K, int64_t ldx, const void* weight, float eps,
                  void* y, void* q, void* scale, int scale_dtype, float* inv_out, hipStream_t st) {
    if (x_dtype != LLMQ_BF16 && x_dtype != LLMQ_F16) return LLMQ_ERR_DTYPE;
    if (M < 0 || K < 0 || ldx < K || (K & 7) || (ldx & 7) || M > 0x7fffffffLL) return LLMQ_ERR_SHAPE;
    if (M == 0) return LLMQ_OK;
    if (K == 0) return LLMQ_ERR_SHAPE;
    if (!x || !weight || (QMODE < 0 ? !y : (!q || !scale))) return LLMQ_ERR_NULL;
    if (QMODE >= 0 && scale_dtype != x_dtype && scale_dtype != LLMQ_F32) return LLMQ_ERR_DTYPE;
    if (!aligned16(x) || !aligned16(weight) || (y && !aligned16(y)) || (q && (reinterpret_cast<uintptr_t>(q) & 7u)))
        return LLMQ_ERR_ALIGN;
    if (x_dtype == LLMQ_BF16)
        return launch_norm<LLMQ_BF16, QMODE>(x, M, K, ldx, weight, eps, y, q, scale, scale_dtype, inv_out, st);
    return launch_norm<LLMQ_F16, QMODE>(x, M, K, ldx, weight, eps, y, q, scale, scale_dtype, inv_out, st);
}

int check_common(const void* x, int x_dtype, int64_t M, int64_t K, int64_t ldx, const void* q) {
    if (!x || !q) return (M == 0 || K == 0) ? LLMQ_OK : LLMQ_ERR_NULL;
    if (x_dtype != LLMQ_BF16 && x_dtype != LLMQ_F16) return LLMQ_ERR_DTYPE;
    if (M < 0 || K < 0 || ldx < K || (K & 7) || (ldx & 7) || M > 0x7fffffffLL) return LLMQ_ERR_SHAPE;
    if (!aligned16(x) || (reinterpret_cast<uintptr_t>(q) & 7u)) return LLMQ_ERR_ALIGN;
    return LLMQ_OK;
}

template <int DT, int MODE, int SCALE>
int launch_rows(const void* x, int64_t M, int64_t K, int64_t ldx, void* q, void* scale, int scale_dtype,
                const float* aux, int n_aux, int static_f32, float floor, hipStream_t st) {
    const dim3 grid((unsigned)M), block(kThreads);
    const uint16_t* xp = (const uint16_t*)x;
    uint8_t* qp = (uint8_t*)q;
    const int64_t per_thread = ((K >> 3) + kThreads - 1) / kThreads;
    if (SCALE == SCALE_ROW && wave_rows(M, K)) {
        const dim3 wgrid((unsigned)((M + kNW - 1) / kNW));
        const int64_t per_lane = ((K >> 3) + kWave - 1) / kWave;
#define LLMQ_LAUNCH_NCW(NCW) \
    hipLaunchKernelGGL((quant_rows_wave_kernel<DT, MODE, NCW>), wgrid, block, 0, st, xp, ldx, K, M, qp, scale, scale_dtype, floor)
        if (per_lane <= 1) LLMQ_LAUNCH_NCW(1);
        else LLMQ_LAUNCH_NCW(2);
#undef LLMQ_LAUNCH_NCW
        return launch_status();
    }
#define LLMQ_LAUNCH_NCT(NC, NT) \
    hipLaunchKernelGGL((quant_rows_kernel<DT, MODE, SCALE, NC, NT>), grid, dim3(NT), 0, st, xp, ldx, K, qp, scale, scale_dtype, aux, n_aux, static_f32, floor)
#define LLMQ_LAUNCH_NC(NC) LLMQ_LAUNCH_NCT(NC, kThreads)
    if (SCALE != SCALE_ROW) LLMQ_LAUNCH_NC(0);
    else if (half_blocks(M, K)) LLMQ_LAUNCH_NCT(4, kThreads / 2);
    else if (per_thread <= 1) LLMQ_LAUNCH_NC(1);
    else if (per_thread <= 2) LLMQ_LAUNCH_NC(2);
    else if (per_thread <= 4) LLMQ_LAUNCH_NC(4);
    else if (per_thread <= 10) LLMQ_LAUNCH_NC(10);
    else LLMQ_LAUNCH_NC(0);
#undef LLMQ_LAUNCH_NC
    return launch_status();
}

template <int MODE, int SCALE>
int dispatch_rows(const void* x, int x_dtype, int64_t M, int64_t K, int64_t ldx, void* q, void* scale,
                  int scale_dtype, const float* aux, int n_aux, int static_f32, float floor, hipStream_t st) {
    if (x_dtype == LLMQ_BF16)
        return launch_rows<LLMQ_BF16, MODE, SCALE>(x, M, K, ldx, q, scale, scale_dtype, aux, n_aux, static_f32, floor, st);
    return launch_rows<LLMQ_F16, MODE, SCALE>(x, M, K, ldx, q, scale, scale_dtype, aux, n_aux, static_f32, floor, st);
}

template <int MODE>
int per_tensor(const void* x, int x_dtype, int64_t M, int64_t K, int64_t ldx, void* q, void* scale,
               int scale_dtype, void* ws, size_t ws_bytes, float floor, hipStream_t st) {
    if (!ws || ws_bytes < kMaxPartials * sizeof(float)) return LLMQ_ERR_WORKSPACE;
    const int64_t total = M * (K >> 3);
    int nblk = (int)((total + kThreads * 4 - 1) / (kThreads * 4));
    nblk = nblk < 1 ? 1 : (nblk > kMaxPartials ? kMaxPartials : nblk);
    float* partials = (float*)ws;
    if (x_dtype == LLMQ_BF16)
        hipLaunchKernelGGL((absmax_partials_kernel<LLMQ_BF16>), dim3(nblk), dim3(kThreads), 0, st,
                           (const uint16_t*)x, ldx, M, K, partials);
    else
        hipLaunchKernelGGL((absmax_partials_kernel<LLMQ_F16>), dim3(nblk), dim3(kThreads), 0, st,
                           (const uint16_t*)x, ldx, M, K, partials);
    if (launch_status() != LLMQ_OK) return LLMQ_ERR_LAUNCH;
    return dispatch_rows<MODE, SCALE_TENSOR>(x, x_dtype, M, K, ldx, q, scale, scale_dtype, partials, nblk, 0, floor, st);
}

// Per-output-channel int8 weight quantizer (an offline step: one pass when a module is built).  One block per
// row of W [N, K]; any K, any 16-bit or fp32 dtype; arithmetic in the dtype of W as the reference's tensor ops do on
// the GPU: scale = round_dt(absmax / 127) with no floor (an all-zero row gives 0 / 0 = NaN, which narrows to 0),
// q = clamp(rint(round_dt(w / scale)), -128, 127), true division.
template <int DT>
__device__ __forceinline__ float wq_load(const void* w, int64_t i) {
    if (DT == LLMQ_F32) return reinterpret_cast<const float*>(w)[i];
    return Lo<DT == LLMQ_F32 ? LLMQ_BF16 : DT>::to_f32(reinterpret_cast<const uint16_t*>(w)[i]);
}
template <int DT>
__device__ __forceinline__ float wq_round(float v) {
    if (DT == LLMQ_F32) return v;
    return Lo<DT == LLMQ_F32 ? LLMQ_BF16 : DT>::round(v);
}
template <int DT>
__global__ __launch_bounds__(kThreads) void quant_weight_rows_kernel(const void* __restrict__ w, int64_t ldw, int64_t K,
                                                                      int8_t* __restrict__ q, void* __restrict__ scale_out) {
    __shared__ float smem[kNW];
    const int64_t row = blockIdx.x;
    float amax = 0.f;
    for (int64_t k = threadIdx.x; k < K; k += kThreads) amax = max_nonneg(amax, fabsf(wq_load<DT>(w, row * ldw + k)));
    const float m = block_max<kNW>(amax, smem);  // NaN if the row holds one, as torch's max
    const float s = wq_round<DT>(m / 127.f);
    if (threadIdx.x == 0) {
        if (DT == LLMQ_F32) reinterpret_cast<float*>(scale_out)[row] = s;
        else reinterpret_cast<uint16_t*>(scale_out)[row] = Lo<DT == LLMQ_F32 ? LLMQ_BF16 : DT>::from_f32(s);
    }
    for (int64_t k = threadIdx.x; k < K; k += kThreads) {
        const float t = wq_round<DT>(wq_load<DT>(w, row * ldw + k) / s);
        const float r = __builtin_rintf(t);
        q[row * K + k] = (t != t) ? (int8_t)0 : (int8_t)__builtin_amdgcn_fmed3f(r, -128.f, 127.f);
    }
}

}  // namespace
}  // namespace llmq

using namespace llmq;

extern "C" size_t llmq_quant_workspace_bytes(void) { return kMaxPartials * sizeof(float); }

extern "C" int llmq_quant_i8_per_token(const void* x, int x_dtype, int64_t M, int64_t K, int64_t ldx,
                                       int8_t* q, void* scale, int scale_dtype, llmq_stream_t stream) {
    return llmq_quant_i8_per_token_floor(x, x_dtype, M, K, ldx, q, scale, scale_dtype, QP<MODE_I8>::floor_, stream);
}

extern "C" int llmq_quant_i8_per_token_floor(const void* x, int x_dtype, int64_t M, int64_t K, int64_t ldx,
                                             int8_t* q, void* scale, int scale_dtype, float absmax_floor,
                                             llmq_stream_t stream) {
    if (!(absmax_floor >= 0.f)) return LLMQ_ERR_SHAPE;
    int rc = check_common(x, x_dtype, M, K, ldx, q);
    if (rc != LLMQ_OK) return rc;
    if (M == 0) return LLMQ_OK;
    if (!scale) return LLMQ_ERR_NULL;
    if (scale_dtype != x_dtype && scale_dtype != LLMQ_F32) return LLMQ_ERR_DTYPE;
    if (K == 0) return LLMQ_ERR_SHAPE;
    return dispatch_rows<MODE_I8, SCALE_ROW>(x, x_dtype, M, K, ldx, q, scale, scale_dtype, nullptr, 0, 0, absmax_floor,
                                             (hipStream_t)stream);
}

extern "C" int llmq_quant_i8_per_tensor(const void* x, int x_dtype, int64_t M, int64_t K, int64_t ldx,
                                        int8_t* q, void* scale, int scale_dtype, void* workspace,
                                        size_t workspace_bytes, llmq_stream_t stream) {
    return llmq_quant_i8_per_tensor_floor(x, x_dtype, M, K, ldx, q, scale, scale_dtype, QP<MODE_I8>::floor_, workspace,
                                          workspace_bytes, stream);
}

extern "C" int llmq_quant_i8_per_tensor_floor(const void* x, int x_dtype, int64_t M, int64_t K, int64_t ldx,
                                              int8_t* q, void* scale, int scale_dtype, float absmax_floor,
                                              void* workspace, size_t workspace_bytes, llmq_stream_t stream) {
    if (!(absmax_floor >= 0.f)) return LLMQ_ERR_SHAPE;
    int rc = check_common(x, x_dtype, M, K, ldx, q);
    if (rc != LLMQ_OK) return rc;
    if (!scale) return LLMQ_ERR_NULL;
    if (scale_dtype != x_dtype && scale_dtype != LLMQ_F32) return LLMQ_ERR_DTYPE;
    if (M == 0 || K == 0) return LLMQ_ERR_SHAPE;
    return per_tensor<MODE_I8>(x, x_dtype, M, K, ldx, q, scale, scale_dtype, workspace, workspace_bytes, absmax_floor,
                               (hipStream_t)stream);
}

extern "C" int llmq_quant_fp8_per_token(const void* x, int x_dtype, int64_t M, int64_t K, int64_t ldx,
                                        uint8_t* q, float* scale, llmq_stream_t stream) {
    int rc = check_common(x, x_dtype, M, K, ldx, q);
    if (rc != LLMQ_OK) return rc;
    if (M == 0) return LLMQ_OK;
    if (!scale) return LLMQ_ERR_NULL;
    if (K == 0) return LLMQ_ERR_SHAPE;
    return dispatch_rows<MODE_F8, SCALE_ROW>(x, x_dtype, M, K, ldx, q, scale, LLMQ_F32, nullptr, 0, 0,
                                             QP<MODE_F8>::floor_, (hipStream_t)stream);
}

extern "C" int llmq_quant_fp8_per_tensor(const void* x, int x_dtype, int64_t M, int64_t K, int64_t ldx,
                                         uint8_t* q, float* scale, void* workspace, size_t workspace_bytes,
                                         llmq_stream_t stream) {
    int rc = check_common(x, x_dtype, M, K, ldx, q);
    if (rc != LLMQ_OK) return rc;
    if (!scale) return LLMQ_ERR_NULL;
    if (M == 0 || K == 0) return LLMQ_ERR_SHAPE;
    return per_tensor<MODE_F8>(x, x_dtype, M, K, ldx, q, scale, LLMQ_F32, workspace, workspace_bytes,
                               QP<MODE_F8>::floor_, (hipStream_t)stream);
}

extern "C" int llmq_quant_fp8_static(const void* x, int x_dtype, int64_t M, int64_t K, int64_t ldx,
                                     uint8_t* q, const float* scale, int scale_is_f32_tensor,
                                     llmq_stream_t stream) {
    int rc = check_common(x, x_dtype, M, K, ldx, q);
    if (rc != LLMQ_OK) return rc;
    if (M == 0 || K == 0) return LLMQ_OK;
    if (!scale) return LLMQ_ERR_NULL;
    return dispatch_rows<MODE_F8, SCALE_STATIC>(x, x_dtype, M, K, ldx, q, nullptr, LLMQ_F32, scale, 1,
                                                scale_is_f32_tensor ? 1 : 0, 0.f, (hipStream_t)stream);
}

extern "C" int llmq_quant_i8_weight_per_channel(const void* w, int w_dtype, int64_t N, int64_t K, int64_t ldw,
                                                int8_t* q, void* scale, llmq_stream_t stream) {
    if (w_dtype != LLMQ_BF16 && w_dtype != LLMQ_F16 && w_dtype != LLMQ_F32) return LLMQ_ERR_DTYPE;
    if (N < 0 || K < 0 || ldw < K || N > 0x7fffffffLL) return LLMQ_ERR_SHAPE;
    if (N == 0) return LLMQ_OK;
    if (K == 0) return LLMQ_ERR_SHAPE;
    if (!w || !q || !scale) return LLMQ_ERR_NULL;
    const dim3 grid((unsigned)N), block(kThreads);
    hipStream_t st = (hipStream_t)stream;
    if (w_dtype == LLMQ_BF16) hipLaunchKernelGGL((quant_weight_rows_kernel<LLMQ_BF16>), grid, block, 0, st, w, ldw, K, q, scale);
    else if (w_dtype == LLMQ_F16) hipLaunchKernelGGL((quant_weight_rows_kernel<LLMQ_F16>), grid, block, 0, st, w, ldw, K, q, scale);
    else hipLaunchKernelGGL((quant_weight_rows_kernel<LLMQ_F32>), grid, block, 0, st, w, ldw, K, q, scale);
    return launch_status();
}

extern "C" int llmq_rmsnorm(const void* x, int x_dtype, int64_t M, int64_t K, int64_t ldx, const void* weight,
                            float eps, void* y, float* inv_rms, llmq_stream_t stream) {
    return rmsnorm_entry<-1>(x, x_dtype, M, K, ldx, weight, eps, y, nullptr, nullptr, LLMQ_F32, inv_rms,
                             (hipStream_t)stream);
}

extern "C" int llmq_rmsnorm_quant_i8_per_token(const void* x, int x_dtype, int64_t M, int64_t K, int64_t ldx,
                                               const void* weight, float eps, void* y, int8_t* q, void* scale,
                                               int scale_dtype, float* inv_rms, llmq_stream_t stream) {
    return rmsnorm_entry<MODE_I8>(x, x_dtype, M, K, ldx, weight, eps, y, q, scale, scale_dtype, inv_rms,
                                  (hipStream_t)stream);
}

extern "C" int llmq_rmsnorm_quant_fp8_per_token(const void* x, int x_dtype, int64_t M, int64_t K, int64_t ldx,
                                                const void* weight, float eps, void* y, uint8_t* q, float* scale,
                                                float* inv_rms, llmq_stream_t stream) {
    return rmsnorm_entry<MODE_F8>(x, x_dtype, M, K, ldx, weight, eps, y, q, scale, LLMQ_F32, inv_rms,
                                  (hipStream_t)stream);
}
