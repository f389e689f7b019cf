// Arithmetic of the activation quantizers (int8 SmoothQuant, OCP e4m3fn FP8), shared by the row kernels (quant.hip)
// and the few-token linear that quantizes on the fly (linear_fused.hip), so that both produce the same bits.
#ifndef LLMQ_QUANT_MATH_H_
#define LLMQ_QUANT_MATH_H_

#include "llmq_common.h"

namespace llmq {
namespace {

enum { MODE_I8 = 0, MODE_F8 = 1 };

template <int MODE> struct QP;
template <> struct QP<MODE_I8> { static constexpr float floor_ = 1e-5f, qmax = 127.f, lo = -128.f, hi = 127.f; };
template <> struct QP<MODE_F8> { static constexpr float floor_ = 1e-12f, qmax = 448.f, lo = -448.f, hi = 448.f; };

// floor: the lower clamp bound of the absmax (1e-5 / 1e-12 in the Linear modules' quantizers, 1e-8 in the reference's
// utils/quantization_utils.py:57-71); it lives in the activation dtype, like every other value of the chain.
template <int DT, int MODE>
__device__ __forceinline__ float scale_from_amax(float amax, float floor = QP<MODE>::floor_) {
    const float fl = Lo<DT>::round(floor);
    return Lo<DT>::round(max_nonneg(amax, fl) / QP<MODE>::qmax);  // a NaN absmax stays NaN, as under torch.clamp
}

typedef uint16_t u16x2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ float absmax8(uint4 r, int dt_is_bf16) {
    // |x| of 8 packed 16-bit floats.  With the sign bits cleared the bit patterns of bf16 / fp16 values
    // order like the values themselves, so the maximum is taken on packed unsigned 16-bit integers
    // (two elements per instruction) and only the winner is widened to fp32.  A NaN pattern is above every number's, so
    // a chunk that holds one returns NaN.
    const u16x2 a = __builtin_bit_cast(u16x2, r.x & 0x7fff7fffu), b = __builtin_bit_cast(u16x2, r.y & 0x7fff7fffu);
    const u16x2 c = __builtin_bit_cast(u16x2, r.z & 0x7fff7fffu), d = __builtin_bit_cast(u16x2, r.w & 0x7fff7fffu);
    const u16x2 m = __builtin_elementwise_max(__builtin_elementwise_max(a, b), __builtin_elementwise_max(c, d));
    const uint16_t top = m[0] > m[1] ? m[0] : m[1];
    return dt_is_bf16 ? __uint_as_float((uint32_t)top << 16) : Lo<LLMQ_F16>::to_f32(top);
}

// Quotient rounded to the activation dtype.  bf16: x * (1/s) rounds to the same bf16 value
// as the exact quotient for every pair of bf16 operands (the exact quotient of two 8-bit
// significands is never closer than 2^-17 relative to a bf16 rounding boundary), so one
// multiply replaces the division.  fp16 significands are too long for that: true division.
// Q_DT: scale is itself a value of the activation dtype (dynamic quantizers).
// Q_DIV_DT: arbitrary fp32 scale, quotient rounded to the activation dtype (tensor / Python float).
// Q_DIV_F32: arbitrary fp32 scale, quotient kept in fp32 (tensor / fp32 tensor promotes).
enum { Q_DT = 0, Q_DIV_DT = 1, Q_DIV_F32 = 2 };
template <int DT, int QUOT>
__device__ __forceinline__ float quotient(float x, float s, float inv_s) {
    if (QUOT == Q_DIV_F32) return x / s;
    if (QUOT == Q_DIV_DT || DT == LLMQ_F16) return Lo<DT>::round(x / s);
    return Lo<DT>::round(x * inv_s);
}
// the quotients of a pair of elements; the two roundings to the activation dtype share one packed conversion
template <int DT, int QUOT>
__device__ __forceinline__ void quotient2(float x0, float x1, float s, float inv_s, float& q0, float& q1) {
    if (QUOT == Q_DIV_F32) {
        q0 = x0 / s, q1 = x1 / s;
        return;
    }
    const bool mul = !(QUOT == Q_DIV_DT || DT == LLMQ_F16);
    const uint32_t p = Lo<DT>::pack2(mul ? x0 * inv_s : x0 / s, mul ? x1 * inv_s : x1 / s);
    q0 = Lo<DT>::lo_f32(p), q1 = Lo<DT>::hi_f32(p);
}

// FIN: the caller knows that no quotient can be NaN (the row's absmax, reduced so that a NaN element makes it NaN, is
// finite, so every element is finite, and the scale is positive): the per-element NaN handling, which then never
// fires, is left out.
template <int DT, int MODE, int QUOT, bool FIN = false>
__device__ __forceinline__ uint2 quant8(uint4 raw, float s, float inv_s) {
    const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
    float f[8];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        float q0, q1;
        quotient2<DT, QUOT>(Lo<DT>::lo_f32(w[i]), Lo<DT>::hi_f32(w[i]), s, inv_s, q0, q1);
        f[2 * i] = q0, f[2 * i + 1] = q1;
    }
#pragma unroll
    for (int i = 0; i < 8; i++) {
        const float q = f[i];
        if (MODE == MODE_I8) {
            f[i] = (!FIN && q != q) ? 0.f : q;  // NaN narrows to 0 (what the reference's cast gives); clamp: see below
        } else {
            const float c = __builtin_amdgcn_fmed3f(q, QP<MODE>::lo, QP<MODE>::hi);
            f[i] = (!FIN && q != q) ? q : c;  // clamp keeps NaN, as torch.clamp does
        }
    }
    uint32_t out[2];
    if (MODE == MODE_I8) {
#pragma unroll
        for (int h = 0; h < 2; h++) {
            // v_cvt_pk_u8_f32 rounds to the nearest integer (ties to even), saturates to [0, 255] and
            // inserts the byte: with the value biased by 128 that is round + clamp(-128, 127) + pack in
            // one instruction per element; the bias is taken out again by flipping the top bit of each byte
            uint32_t w = 0;
#pragma unroll
            for (int i = 0; i < 4; i++) w = __builtin_amdgcn_cvt_pk_u8_f32(f[4 * h + i] + 128.0f, i, w);
            out[h] = w ^ 0x80808080u;
        }
    } else {
#pragma unroll
        for (int h = 0; h < 2; h++) {
            int p = 0;
            p = __builtin_amdgcn_cvt_pk_fp8_f32(f[4 * h + 0], f[4 * h + 1], p, false);
            p = __builtin_amdgcn_cvt_pk_fp8_f32(f[4 * h + 2], f[4 * h + 3], p, true);
            out[h] = (uint32_t)p;
        }
    }
    return make_uint2(out[0], out[1]);
}

}  // namespace
}  // namespace llmq

#endif  // LLMQ_QUANT_MATH_H_
