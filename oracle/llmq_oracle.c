/* Scalar C restatement of the reference's quantized-linear arithmetic.
 *
 * TEST INFRASTRUCTURE ONLY: loaded by tests/, by __graft_entry__.smoke() and by the
 * cpu_baseline leg of bench.py as the checker; never linked into or called from the
 * product library.  It is written independently of oracle/ref_math.py (explicit bit
 * manipulation instead of torch's dtype machinery) so that agreement between the two is a
 * real check of both.  Reference citations are relative to the reference's runtime/ dir.
 *
 * Build: oracle/build_oracle.py (gcc -O2 -shared -fPIC, no -ffast-math).
 */
#include <math.h>
#include <stdint.h>
#include <string.h>

enum { ORC_BF16 = 0, ORC_F16 = 1 };

static float bits_f32(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }
static uint32_t f32_bits(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }

/* ---- bf16 ---- */
static float bf16_to_f32(uint16_t h) { return bits_f32((uint32_t)h << 16); }
static uint16_t f32_to_bf16(float f) {           /* round to nearest even */
    uint32_t u = f32_bits(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40); /* quiet NaN */
    uint32_t lsb = (u >> 16) & 1u;
    u += 0x7fffu + lsb;
    return (uint16_t)(u >> 16);
}

/* ---- fp16 ---- */
static float f16_to_f32(uint16_t h) {
    uint32_t s = (uint32_t)(h & 0x8000u) << 16, e = (h >> 10) & 0x1f, m = h & 0x3ff;
    if (e == 0) {
        if (m == 0) return bits_f32(s);
        float v = ldexpf((float)m, -24);
        return s ? -v : v;
    }
    if (e == 31) return bits_f32(s | 0x7f800000u | (m << 13));
    return bits_f32(s | ((e + 112) << 23) | (m << 13));
}
static uint16_t f32_to_f16(float f) {            /* round to nearest even, IEEE overflow -> inf */
    uint32_t u = f32_bits(f), s = (u >> 16) & 0x8000u, a = u & 0x7fffffffu;
    if (a > 0x7f800000u) return (uint16_t)(s | 0x7e00);
    if (a >= 0x477ff000u) return (uint16_t)(s | 0x7c00);      /* >= 65520 rounds to inf */
    if (a < 0x33000001u) return (uint16_t)s;                   /* <= 2^-25 rounds to 0 */
    int e = (int)(a >> 23) - 127;
    uint32_t m = (a & 0x7fffffu) | 0x800000u;                  /* 24-bit significand */
    int shift = (e < -14) ? (13 + (-14 - e)) : 13;             /* bits to drop */
    uint32_t keep = m >> shift, rem = m & ((1u << shift) - 1), half = 1u << (shift - 1);
    if (rem > half || (rem == half && (keep & 1u))) keep++;
    if (e < -14) return (uint16_t)(s | keep);                  /* subnormal (may carry to normal) */
    return (uint16_t)(s | (((uint32_t)(e + 15) << 10) + (keep - 0x400u)));
}

static float lo_to_f32(uint16_t h, int dt) { return dt == ORC_BF16 ? bf16_to_f32(h) : f16_to_f32(h); }
static uint16_t f32_to_lo(float f, int dt) { return dt == ORC_BF16 ? f32_to_bf16(f) : f32_to_f16(f); }

uint16_t orc_f32_to_bf16(float f) { return f32_to_bf16(f); }
uint16_t orc_f32_to_f16(float f) { return f32_to_f16(f); }
float orc_f16_to_f32(uint16_t h) { return f16_to_f32(h); }

/* ---- OCP e4m3fn ---- */
float orc_e4m3_decode(uint8_t c) {
    int s = c >> 7, e = (c >> 3) & 0xf, m = c & 7;
    float v;
    if (e == 15 && m == 7) return NAN;
    if (e == 0) v = ldexpf((float)m, -9);             /* subnormal: m * 2^-6 / 8 */
    else v = ldexpf((float)(8 + m), e - 10);          /* (1 + m/8) * 2^(e-7) */
    return s ? -v : v;
}
/* Round-to-nearest-even encode with torch's cast semantics: |x| beyond the largest value
 * that still rounds to 448 (464 is a tie that goes to even = 448) becomes NaN (0x7f). */
uint8_t orc_e4m3_encode(float f) {
    uint32_t u = f32_bits(f);
    uint8_t s = (uint8_t)((u >> 24) & 0x80);
    float a = fabsf(f);
    if (!(a == a)) return (uint8_t)(s | 0x7f);
    if (a > 464.0f) return (uint8_t)(s | 0x7f);
    if (a >= 448.0f) return (uint8_t)(s | 0x7e);
    if (a < ldexpf(1.0f, -6)) {                        /* subnormal range: step 2^-9 */
        float q = rintf(a * 512.0f);                   /* exact scaling, half-to-even */
        return (uint8_t)(s | (uint8_t)q);              /* q == 8 encodes 2^-6 (e=1, m=0) */
    }
    int e; float fr = frexpf(a, &e);                   /* a = fr * 2^e, fr in [0.5, 1) */
    float q = rintf(fr * 16.0f);                       /* 8..16 */
    if (q == 16.0f) { q = 8.0f; e++; }
    int be = e - 1 + 7;
    return (uint8_t)(s | (be << 3) | ((int)q - 8));
}

/* ---- int8 quantizers: nn_models/modules/linear/linear_sq.py:44-65 ---- */
static int8_t quant_one_i8(uint16_t xb, float scale_f, int dt) {
    float q = lo_to_f32(f32_to_lo(lo_to_f32(xb, dt) / scale_f, dt), dt);  /* quotient rounded to x dtype */
    float r = rintf(q);
    if (!(r == r)) return 0;
    if (r < -128.0f) r = -128.0f;
    if (r > 127.0f) r = 127.0f;
    return (int8_t)r;
}
static uint16_t scale_from_amax(float amax, float floor_, float qmax, int dt) {
    float fl = lo_to_f32(f32_to_lo(floor_, dt), dt);  /* the clamp bound is rounded to x dtype */
    if (amax < fl) amax = fl;
    return f32_to_lo(amax / qmax, dt);
}
void orc_quant_i8_per_token(const uint16_t* x, int dt, long M, long K, int8_t* q, uint16_t* scale) {
    for (long m = 0; m < M; m++) {
        float amax = 0.f;
        for (long k = 0; k < K; k++) { float v = fabsf(lo_to_f32(x[m * K + k], dt)); if (v > amax) amax = v; }
        uint16_t sb = scale_from_amax(amax, 1e-5f, 127.f, dt);
        scale[m] = sb;
        float sf = lo_to_f32(sb, dt);
        for (long k = 0; k < K; k++) q[m * K + k] = quant_one_i8(x[m * K + k], sf, dt);
    }
}
void orc_quant_i8_per_tensor(const uint16_t* x, int dt, long n, int8_t* q, uint16_t* scale) {
    float amax = 0.f;
    for (long i = 0; i < n; i++) { float v = fabsf(lo_to_f32(x[i], dt)); if (v > amax) amax = v; }
    uint16_t sb = scale_from_amax(amax, 1e-5f, 127.f, dt);
    *scale = sb;
    float sf = lo_to_f32(sb, dt);
    for (long i = 0; i < n; i++) q[i] = quant_one_i8(x[i], sf, dt);
}

/* ---- fp8 quantizers: nn_models/modules/linear/linear_fp8.py:11-63 ---- */
static uint8_t quant_one_f8(uint16_t xb, float scale_f, int dt) {
    float q = lo_to_f32(f32_to_lo(lo_to_f32(xb, dt) / scale_f, dt), dt);
    if (q < -448.f) q = -448.f;
    if (q > 448.f) q = 448.f;
    return orc_e4m3_encode(q);
}
void orc_quant_fp8_per_token(const uint16_t* x, int dt, long M, long K, uint8_t* q, float* scale) {
    for (long m = 0; m < M; m++) {
        float amax = 0.f;
        for (long k = 0; k < K; k++) { float v = fabsf(lo_to_f32(x[m * K + k], dt)); if (v > amax) amax = v; }
        float sf = lo_to_f32(scale_from_amax(amax, 1e-12f, 448.f, dt), dt);
        scale[m] = sf;
        for (long k = 0; k < K; k++) q[m * K + k] = quant_one_f8(x[m * K + k], sf, dt);
    }
}
void orc_quant_fp8_per_tensor(const uint16_t* x, int dt, long n, uint8_t* q, float* scale) {
    float amax = 0.f;
    for (long i = 0; i < n; i++) { float v = fabsf(lo_to_f32(x[i], dt)); if (v > amax) amax = v; }
    float sf = lo_to_f32(scale_from_amax(amax, 1e-12f, 448.f, dt), dt);
    *scale = sf;
    for (long i = 0; i < n; i++) q[i] = quant_one_f8(x[i], sf, dt);
}

/* ---- exact int8 GEMM: csrc/smoothquant/sq_gemm.cu:67-76 (A [M,K] row-major, B [N,K]) ---- */
void orc_gemm_i8(const int8_t* A, const int8_t* B, long M, long N, long K, int32_t* acc) {
    for (long m = 0; m < M; m++)
        for (long n = 0; n < N; n++) {
            int64_t s = 0;
            for (long k = 0; k < K; k++) s += (int64_t)A[m * K + k] * (int64_t)B[n * K + k];
            acc[m * N + n] = (int32_t)s;
        }
}

/* ---- AWQ: utils/packing_utils.py:4-80 ---- */
static const int REV[8] = {0, 4, 1, 5, 2, 6, 3, 7};
/* out fp16 bits [K, N] */
void orc_awq_dequant(const int32_t* qweight, const int32_t* qzeros, const uint16_t* scales,
                     long K, long N, long G, uint16_t* out) {
    long Nw = N / 8;
    for (long k = 0; k < K; k++)
        for (long n = 0; n < N; n++) {
            uint32_t w = (uint32_t)qweight[k * Nw + n / 8], z = (uint32_t)qzeros[(k / G) * Nw + n / 8];
            int sh = 4 * REV[n % 8];
            int d = (int)((w >> sh) & 0xf) - (int)((z >> sh) & 0xf);
            float p = (float)d * f16_to_f32(scales[(k / G) * N + n]);   /* exact in fp32 */
            out[k * N + n] = f32_to_f16(p);
        }
}
/* x fp16 [M,K] times dequantized W [K,N], double accumulation, fp16 result */
void orc_awq_gemm(const uint16_t* x, const int32_t* qweight, const int32_t* qzeros,
                  const uint16_t* scales, long M, long N, long K, long G, uint16_t* out) {
    long Nw = N / 8;
    for (long m = 0; m < M; m++)
        for (long n = 0; n < N; n++) {
            double s = 0.0;
            int sh = 4 * REV[n % 8];
            for (long k = 0; k < K; k++) {
                uint32_t w = (uint32_t)qweight[k * Nw + n / 8], z = (uint32_t)qzeros[(k / G) * Nw + n / 8];
                int d = (int)((w >> sh) & 0xf) - (int)((z >> sh) & 0xf);
                float wv = f16_to_f32(f32_to_f16((float)d * f16_to_f32(scales[(k / G) * N + n])));
                s += (double)f16_to_f32(x[m * K + k]) * (double)wv;
            }
            out[m * N + n] = f32_to_f16((float)s);
        }
}

/* ---- RMSNorm given the reciprocal RMS (nn_models/modules/nonlinear/norm.py:14-16):
 * y = round_dt(w * round_dt(fp32(x) * inv)), scalar loops. */
void orc_rmsnorm_given_inv(const uint16_t* x, const uint16_t* w, const float* inv, int dt, long M, long K,
                           uint16_t* y) {
    for (long m = 0; m < M; m++)
        for (long k = 0; k < K; k++) {
            const float n = lo_to_f32(f32_to_lo(lo_to_f32(x[m * K + k], dt) * inv[m], dt), dt);
            y[m * K + k] = f32_to_lo(lo_to_f32(w[k], dt) * n, dt);
        }
}

/* Reciprocal RMS with the mean accumulated in double (the value every fp32 summation order approximates). */
void orc_inv_rms_f64(const uint16_t* x, int dt, long M, long K, double eps, double* inv) {
    for (long m = 0; m < M; m++) {
        double ss = 0.0;
        for (long k = 0; k < K; k++) {
            const double h = (double)lo_to_f32(x[m * K + k], dt);
            ss += h * h;
        }
        inv[m] = 1.0 / sqrt(ss / (double)K + eps);
    }
}
