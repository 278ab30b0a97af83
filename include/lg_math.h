/* lg_math.h — the elementary functions of the verify path, defined once.
 *
 * The reference leaves expf/tanhf/cosf/sinf to whatever libm the backend links
 * (host glibc in src/cpu/model-cpu.c:87-119, the CUDA device library in
 * src/cuda/model-cuda.cuh:309-324,527-608,663-701), so its CPU and GPU backends
 * agree only to a few ulp.  This build pins them instead: every function below is
 * a fixed sequence of IEEE-754 binary32 add / mul / fma / div / rint operations
 * and integer bit moves, so a host compiler (built with -ffp-contract=off and a
 * hardware fma) and hipcc for gfx950 (same flag, correctly rounded divide/sqrt)
 * produce the same bits.  The HIP kernels and the CPU oracle both include this
 * header; tests pin each function against double-precision libm within a few ulp.
 *
 * Nothing here may be "optimised" on one side only: changing an operation order
 * changes results in the last bit and breaks bit-parity between GPU and oracle.
 */
#ifndef LG_MATH_H
#define LG_MATH_H

#include <stdint.h>

#if defined(__HIPCC__)
#define LG_HD __host__ __device__ static inline
#else
#define LG_HD static inline
#endif

LG_HD float lg_fmaf(float a, float b, float c) { return __builtin_fmaf(a, b, c); }
LG_HD float lg_rintf(float x) { return __builtin_rintf(x); }      /* ties to even */
LG_HD float lg_fabsf(float x) { return __builtin_fabsf(x); }

LG_HD float lg_bits_to_f32(uint32_t u) {
    union { uint32_t u; float f; } c; c.u = u; return c.f;
}
LG_HD uint32_t lg_f32_to_bits(float f) {
    union { uint32_t u; float f; } c; c.f = f; return c.u;
}

/* e^x for x <= 88.  Range reduction x = n ln2 + r with a two-constant split of
 * ln2, degree-6 polynomial on |r| <= ln2/2, scaling by 2^n through the exponent
 * field.  Inputs below -87 return 0 (the softmax tail), so no subnormal scale. */
LG_HD float lg_expf(float x) {
    if (x < -87.0f) return 0.0f;
    if (x > 88.0f) x = 88.0f;
    float n = lg_rintf(x * 1.44269504088896341f);
    float r = lg_fmaf(n, -0.693145751953125f, x);
    r = lg_fmaf(n, -1.428606765330187045e-06f, r);
    float p = 1.9875691500e-4f;
    p = lg_fmaf(p, r, 1.3981999507e-3f);
    p = lg_fmaf(p, r, 8.3334519073e-3f);
    p = lg_fmaf(p, r, 4.1665795894e-2f);
    p = lg_fmaf(p, r, 1.6666665459e-1f);
    p = lg_fmaf(p, r, 5.0000001201e-1f);
    float y = lg_fmaf(p, r * r, r) + 1.0f;
    int32_t ni = (int32_t)n;
    return y * lg_bits_to_f32((uint32_t)(ni + 127) << 23);
}

/* tanh(x): odd polynomial below 0.625, 1 - 2/(e^{2|x|}+1) above, +-1 past 9. */
LG_HD float lg_tanhf(float x) {
    float ax = lg_fabsf(x);
    if (ax < 0.625f) {
        float z = x * x;
        float p = -5.70498872745e-3f;
        p = lg_fmaf(p, z, 2.06390887954e-2f);
        p = lg_fmaf(p, z, -5.37397155531e-2f);
        p = lg_fmaf(p, z, 1.33314422036e-1f);
        p = lg_fmaf(p, z, -3.33332819422e-1f);
        return lg_fmaf(p * z, x, x);
    }
    float t;
    if (ax > 9.0f) t = 1.0f;
    else {
        float e = lg_expf(ax + ax);
        t = 1.0f - 2.0f / (e + 1.0f);
    }
    return x < 0.0f ? -t : t;
}

/* sin and cos of x, |x| up to a few 1e5 (rotary angles are position * frequency).
 * Three-constant Cody-Waite reduction by pi/2 with fma, then the usual minimax
 * polynomials on [-pi/4, pi/4] and a quadrant swap. */
LG_HD void lg_sincosf(float x, float *sn, float *cs) {
    float n = lg_rintf(x * 0.636619772367581343f);
    float r = lg_fmaf(n, -1.57079637050628662109375f, x);
    r = lg_fmaf(n, 4.37113900018624283e-8f, r);
    r = lg_fmaf(n, 1.71512449599242e-15f, r);
    float z = r * r;
    float ps = -1.9515295891e-4f;
    ps = lg_fmaf(ps, z, 8.3321608736e-3f);
    ps = lg_fmaf(ps, z, -1.6666654611e-1f);
    float s = lg_fmaf(ps * z, r, r);
    float pc = 2.443315711809948e-5f;
    pc = lg_fmaf(pc, z, -1.388731625493765e-3f);
    pc = lg_fmaf(pc, z, 4.166664568298827e-2f);
    float c = lg_fmaf(pc * z, z, lg_fmaf(-0.5f, z, 1.0f));
    int32_t q = (int32_t)n & 3;
    float so = (q & 1) ? c : s;
    float co = (q & 1) ? s : c;
    if (q == 1 || q == 2) co = -co;
    if (q >= 2) so = -so;
    *sn = so; *cs = co;
}

/* GELU, tanh form, with the reference's constants and evaluation order
 * (src/cpu/model-cpu.c:108-111, src/cuda/model-cuda.cuh:663-666). */
LG_HD float lg_gelu(float x) {
    const float k = 0.7978845608028654f;
    return 0.5f * x * (1.0f + lg_tanhf(k * (x + 0.044715f * x * x * x)));
}

/* binary32 -> binary16, round to nearest even, subnormals and NaN kept
 * (same value as src/cpu/model-cpu.c:185-200 and the device convert). */
LG_HD uint16_t lg_f32_to_f16(float f) {
    uint32_t w = lg_f32_to_bits(f);
    uint32_t sign = (w >> 16) & 0x8000u;
    uint32_t a = w & 0x7FFFFFFFu;
    if (a >= 0x7F800000u)                       /* inf / nan */
        return (uint16_t)(sign | (a > 0x7F800000u ? 0x7E00u : 0x7C00u));
    if (a >= 0x477FF000u)                       /* rounds to >= 65520 -> inf */
        return (uint16_t)(sign | 0x7C00u);
    if (a < 0x33000001u)                        /* <= 2^-25: rounds to zero */
        return (uint16_t)sign;
    uint32_t e = a >> 23;
    uint32_t man = (a & 0x007FFFFFu) | 0x00800000u;
    uint32_t shift = e >= 113 ? 13u : (126u - e);          /* subnormal halves shift more */
    uint32_t half = (e >= 113 ? (e - 112u) << 10 : 0u) + ((man >> shift) & (e >= 113 ? 0x3FFu : 0x7FFu));
    uint32_t rem = man & ((1u << shift) - 1u);
    uint32_t mid = 1u << (shift - 1u);
    if (rem > mid || (rem == mid && (half & 1u))) half++;
    return (uint16_t)(sign | half);
}

LG_HD float lg_f16_to_f32(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t e = (h >> 10) & 0x1Fu, m = h & 0x3FFu;
    if (e == 0) {
        if (m == 0) return lg_bits_to_f32(sign);
        float v = (float)m * 5.9604644775390625e-8f;        /* m * 2^-24, exact */
        return sign ? -v : v;
    }
    if (e == 31) return lg_bits_to_f32(sign | 0x7F800000u | (m << 13));
    return lg_bits_to_f32(sign | ((e + 112u) << 23) | (m << 13));
}

#endif /* LG_MATH_H */
