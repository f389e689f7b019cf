// Shared device/host helpers for the gfx950 kernels of libllmq_gfx950.so.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "llmq.h"

namespace llmq {

constexpr int kWave = 64;  // CDNA wavefront width

// ---- 16-bit float storage types, handled as raw bits + fp32 math -------------------------
template <int DT> struct Lo;
typedef float lo_f2 __attribute__((ext_vector_type(2)));
template <> struct Lo<LLMQ_BF16> {
    static __device__ __forceinline__ float to_f32(uint16_t h) { return __uint_as_float((uint32_t)h << 16); }
    static __device__ __forceinline__ uint16_t from_f32(float f) {  // round to nearest even
        return __builtin_bit_cast(uint16_t, (__bf16)f);
    }
    static __device__ __forceinline__ float round(float f) { return to_f32(from_f32(f)); }
    // two values narrowed by one packed conversion: a in the low half, b in the high half
    static __device__ __forceinline__ uint32_t pack2(float a, float b) {
        typedef __bf16 bf2 __attribute__((ext_vector_type(2)));
        return __builtin_bit_cast(uint32_t, __builtin_convertvector(lo_f2{a, b}, bf2));
    }
    static __device__ __forceinline__ float lo_f32(uint32_t p) { return __uint_as_float(p << 16); }
    static __device__ __forceinline__ float hi_f32(uint32_t p) { return __uint_as_float(p & 0xffff0000u); }
};
template <> struct Lo<LLMQ_F16> {
    static __device__ __forceinline__ float to_f32(uint16_t h) { return (float)__builtin_bit_cast(_Float16, h); }
    static __device__ __forceinline__ uint16_t from_f32(float f) { return __builtin_bit_cast(uint16_t, (_Float16)f); }
    static __device__ __forceinline__ float round(float f) { return to_f32(from_f32(f)); }
    static __device__ __forceinline__ uint32_t pack2(float a, float b) {
        typedef _Float16 h2 __attribute__((ext_vector_type(2)));
        return __builtin_bit_cast(uint32_t, __builtin_convertvector(lo_f2{a, b}, h2));
    }
    static __device__ __forceinline__ float lo_f32(uint32_t p) { return to_f32((uint16_t)(p & 0xffffu)); }
    static __device__ __forceinline__ float hi_f32(uint32_t p) { return to_f32((uint16_t)(p >> 16)); }
};

// GEMM epilogue value in fp32, each node rounded once: (acc * sa) * sw, then one fused multiply-add with alpha and
// the bias term.  The result is made opaque to the compiler before it is converted to the output type: otherwise
// the fma and a conversion to fp16 may or may not be merged into one mixed-precision instruction that rounds the
// exact sum straight to fp16, and two code paths could disagree on ties of the double rounding.
// PLAIN (no bias term and alpha = 1): the scaled accumulator is the result, as in the reference's epilogue without a bias.
template <bool PLAIN = false>
__device__ __forceinline__ float epi_value(float acc, float sa, float sw, float alpha, float bb) {
    float p = (acc * sa) * sw;
    asm volatile("" : "+v"(p));  // the scaled accumulator is a value of its own: never contracted into what follows
    if constexpr (PLAIN) return p;
    float r = fmaf(alpha, p, bb);
    asm volatile("" : "+v"(r));
    return r;
}

// Round trip of a finished output value through e4m3fn on a stored per-tensor scale, the reference's
// `static_per_tensor_quantize(output, output_scale).to(dtype) * output_scale`
// (nn_models/modules/linear/linear_fp8.py:309-311): f is the output already rounded to its 16-bit type; the quotient by
// the fp32 scale is an fp32 division (a tensor / fp32 tensor promotes), clamped with NaN kept, narrowed to e4m3fn
// (round to nearest even), widened again (exact) and multiplied by the scale in fp32.
__device__ __forceinline__ float fp8_round_trip(float f, float s) {
    const float q = f / s;
    const float c = (q != q) ? q : __builtin_amdgcn_fmed3f(q, -448.f, 448.f);
    const int code = __builtin_amdgcn_cvt_pk_fp8_f32(c, c, 0, false);
    return __builtin_amdgcn_cvt_f32_fp8(code, 0) * s;
}

// 16-byte store of finished output with the non-temporal hint: the tile is not read again by this kernel, and
// without the hint its lines are allocated in L2 beside the operand panels the other tiles of the XCD still need
// (measured on 8192 x 37888 x 3584: 1177 -> 1042 us, the same as storing into a cache-resident dummy region).
__device__ __forceinline__ void store_streaming(void* p, uint4 v) {
    typedef uint32_t u4v __attribute__((ext_vector_type(4)));
    __builtin_nontemporal_store(u4v{v.x, v.y, v.z, v.w}, reinterpret_cast<u4v*>(p));
}
__device__ __forceinline__ float load_as_f32(const void* p, int dtype, int64_t i) {
    if (dtype == LLMQ_F32) return ((const float*)p)[i];
    uint16_t h = ((const uint16_t*)p)[i];
    return dtype == LLMQ_BF16 ? Lo<LLMQ_BF16>::to_f32(h) : Lo<LLMQ_F16>::to_f32(h);
}

// ---- wavefront / block reductions ---------------------------------------------------------
// Maximum of two values that are not negative (absolute values, flags), taken on the bit patterns: those order like
// the values, and a NaN (sign bit clear) is above every number, so it survives every step of a reduction the way
// torch's max / amax propagate it; fmaxf would drop it.
__device__ __forceinline__ float max_nonneg(float a, float b) {
    const uint32_t x = __float_as_uint(a), y = __float_as_uint(b);
    return __uint_as_float(x > y ? x : y);
}

// The value of lane (lane ^ O), O a power of two, without an address computation: DPP lane selects inside quads and
// 16-lane rows, ds_swizzle inside 32 lanes, v_permlane32_swap across the two halves of the wavefront.
template <int O>
__device__ __forceinline__ float lane_xor(float v) {
    const int i = __float_as_int(v);
    if constexpr (O == 1) return __int_as_float(__builtin_amdgcn_mov_dpp(i, 0xB1, 0xf, 0xf, true));        // quad_perm [1,0,3,2]
    else if constexpr (O == 2) return __int_as_float(__builtin_amdgcn_mov_dpp(i, 0x4E, 0xf, 0xf, true));   // quad_perm [2,3,0,1]
    else if constexpr (O == 4) return __int_as_float(__builtin_amdgcn_ds_swizzle(i, 0x101F));              // xor_mask 4
    else if constexpr (O == 8) return __int_as_float(__builtin_amdgcn_mov_dpp(i, 0x128, 0xf, 0xf, true));  // row_ror:8
    else {
        static_assert(O == 16, "lane distance");
        return __int_as_float(__builtin_amdgcn_ds_swizzle(i, 0x401F));  // xor_mask 16
    }
}
// Distance 32: v_permlane32_swap of v with itself returns {v with its upper half replaced by its lower half, v with its
// lower half replaced by its upper half}; in every lane one of the two is the lane's own value and the other its partner's.
__device__ __forceinline__ void lane_xor32_pair(float v, float& a, float& b) {
    const auto sw = __builtin_amdgcn_permlane32_swap(__float_as_int(v), __float_as_int(v), false, false);
    a = __int_as_float(sw[0]);
    b = __int_as_float(sw[1]);
}

__device__ __forceinline__ float wave_max(float v) {
    float a, b;
    lane_xor32_pair(v, a, b);
    v = max_nonneg(a, b);
    v = max_nonneg(v, lane_xor<16>(v));
    v = max_nonneg(v, lane_xor<8>(v));
    v = max_nonneg(v, lane_xor<4>(v));
    v = max_nonneg(v, lane_xor<2>(v));
    v = max_nonneg(v, lane_xor<1>(v));
    return v;
}

// max over a block of NW wavefronts (non-negative values, NaN propagates); every thread gets the result.
// `smem` holds NW floats.
template <int NW>
__device__ __forceinline__ float block_max(float v, float* smem) {
    v = wave_max(v);
    const int lane = threadIdx.x & (kWave - 1), w = threadIdx.x / kWave;
    __syncthreads();  // smem may still be read from a previous call
    if (lane == 0) smem[w] = v;
    __syncthreads();
    float r = smem[0];
#pragma unroll
    for (int i = 1; i < NW; i++) r = max_nonneg(r, smem[i]);
    return r;
}

// butterfly: lane distances 32, 16, 8, 4, 2, 1 in this order; every lane ends with the same bits
__device__ __forceinline__ float wave_sum(float v) {
    float a, b;
    lane_xor32_pair(v, a, b);
    v = a + b;  // own value + partner's, in either order
    v += lane_xor<16>(v);
    v += lane_xor<8>(v);
    v += lane_xor<4>(v);
    v += lane_xor<2>(v);
    v += lane_xor<1>(v);
    return v;
}

// sum over a block of NW wavefronts in a fixed order; every thread gets the same result.
template <int NW>
__device__ __forceinline__ float block_sum(float v, float* smem) {
    v = wave_sum(v);
    const int lane = threadIdx.x & (kWave - 1), w = threadIdx.x / kWave;
    __syncthreads();
    if (lane == 0) smem[w] = v;
    __syncthreads();
    float r = smem[0];
#pragma unroll
    for (int i = 1; i < NW; i++) r += smem[i];
    return r;
}

inline int launch_status() { return hipGetLastError() == hipSuccess ? LLMQ_OK : LLMQ_ERR_LAUNCH; }
inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

}  // namespace llmq
