// tanhf, expf and logf as the C library of the reference's platform computes them, bit for bit.
//
// The reference's GMath::squash and GMath::outputNodeCost ("Backend/Machine Learning/GMath/gmath.cpp":
// 22-101, 272-321) call tanh / exp / log on floats, which resolve to the float routines of the C
// library it is linked against.  That library is a dependency outside the reference tree: GNU libc,
// 2.35 on this platform (x86-64).  Its routines are restated here from their published algorithms so
// that the device produces the same float for every input:
//   tanhf  fdlibm's float routine (sysdeps/ieee754/flt-32/s_tanhf.c): 1 - 2/(expm1f(2|x|)+2) for
//          |x| >= 1, -t/(t+2) with t = expm1f(-2|x|) below, all in float arithmetic;
//   expm1f fdlibm's float routine (s_expm1f.c): reduction by k*ln2 (hi + lo), the degree-5 rational
//          correction in x*x/2, reconstruction by cases of k;
//   expf   the table-driven routine (e_expf.c, from ARM's optimized routines): x*32/ln2 = k + r,
//          2^(k/32) from a 32-entry table, a cubic in r, all in double, one rounding to float;
//   logf   the table-driven routine (e_logf.c, same origin): z/c - 1 with c from a 16-entry table, a
//          cubic in r, all in double, one rounding to float.
// expf and logf are written with the fused multiply-adds of the library's FMA build, which is the
// one x86-64 selects at run time on every CPU with FMA; without them expf differs in 2 of the 2^32
// inputs (0x4202422f, 0xc27c65d9) and logf in none.
//
// Checked against the C library over all 2^32 inputs of each function (0 mismatches; NaNs compared as
// NaNs); the committed tests repeat the comparison on a strided subset on the CPU and on the device.
//
// Everything here must be compiled without contraction of the float operations (the functions
// switch it off themselves under clang; gcc needs -ffp-contract=off).  Error conditions return the
// IEEE result; errno and exception flags are not part of this.
#pragma once

#include <stdint.h>

#if defined(__HIPCC__)
#define GLM_FN __host__ __device__ inline
#else
#define GLM_FN static inline
#endif

#if defined(__clang__)
#define GLM_NO_CONTRACT _Pragma("clang fp contract(off)")
#else
#define GLM_NO_CONTRACT
#endif

GLM_FN uint32_t glm_f2u(float f) { return __builtin_bit_cast(uint32_t, f); }
GLM_FN float glm_u2f(uint32_t u) { return __builtin_bit_cast(float, u); }
GLM_FN uint64_t glm_d2u(double f) { return __builtin_bit_cast(uint64_t, f); }
GLM_FN double glm_u2d(uint64_t u) { return __builtin_bit_cast(double, u); }

GLM_FN float glm_expm1f(float x)
{
    GLM_NO_CONTRACT
    const float one = 1.0f, tiny = 1.0e-30f, huge = 1.0e+30f;
    const float o_threshold = 8.8721679688e+01f, ln2_hi = 6.9313812256e-01f, ln2_lo = 9.0580006145e-06f,
                invln2 = 1.4426950216e+00f;
    const float Q1 = -3.3333335072e-02f, Q2 = 1.5873016091e-03f, Q3 = -7.9365076090e-05f, Q4 = 4.0082177293e-06f,
                Q5 = -2.0109921195e-07f;
    float y, hi, lo, c = 0.0f, t, e, hxs, hfx, r1;
    int32_t k;
    uint32_t hx = glm_f2u(x);
    const uint32_t xsb = hx & 0x80000000u;
    hx &= 0x7fffffffu;
    if (hx >= 0x4195b844u) {          // |x| >= 27 ln2
        if (hx >= 0x42b17218u) {      // |x| >= 88.72...
            if (hx > 0x7f800000u) return x + x;
            if (hx == 0x7f800000u) return (xsb == 0) ? x : -1.0f;
            if (x > o_threshold) return huge * huge;
        }
        if (xsb != 0) return tiny - one;
    }
    if (hx > 0x3eb17218u) {           // |x| > 0.5 ln2
        if (hx < 0x3F851592u) {       // |x| < 1.5 ln2
            if (xsb == 0) { hi = x - ln2_hi; lo = ln2_lo; k = 1; }
            else { hi = x + ln2_hi; lo = -ln2_lo; k = -1; }
        } else {
            k = (int32_t)(invln2 * x + ((xsb == 0) ? 0.5f : -0.5f));
            t = (float)k;
            hi = x - t * ln2_hi;
            lo = t * ln2_lo;
        }
        x = hi - lo;
        c = (hi - x) - lo;
    } else if (hx < 0x33000000u) {    // |x| < 2^-25
        t = huge + x;
        return x - (t - (huge + x));
    } else {
        k = 0;
    }
    hfx = 0.5f * x;
    hxs = x * hfx;
    r1 = one + hxs * (Q1 + hxs * (Q2 + hxs * (Q3 + hxs * (Q4 + hxs * Q5))));
    t = 3.0f - r1 * hfx;
    e = hxs * ((r1 - t) / (6.0f - x * t));
    if (k == 0) return x - (x * e - hxs);
    e = (x * (e - c) - c);
    e -= hxs;
    if (k == -1) return 0.5f * (x - e) - 0.5f;
    if (k == 1) {
        if (x < -0.25f) return -2.0f * (e - (x + 0.5f));
        return one + 2.0f * (x - e);
    }
    if (k <= -2 || k > 56) {
        y = one - (e - x);
        y = glm_u2f(glm_f2u(y) + ((uint32_t)k << 23));
        return y - one;
    }
    if (k < 23) {
        t = glm_u2f(0x3f800000u - (0x1000000u >> k));  // 1 - 2^-k
        y = t - (e - x);
        y = glm_u2f(glm_f2u(y) + ((uint32_t)k << 23));
    } else {
        t = glm_u2f((uint32_t)(0x7f - k) << 23);        // 2^-k
        y = x - (e + t);
        y += one;
        y = glm_u2f(glm_f2u(y) + ((uint32_t)k << 23));
    }
    return y;
}

GLM_FN float glm_tanhf(float x)
{
    GLM_NO_CONTRACT
    const float one = 1.0f, two = 2.0f, tiny = 1.0e-30f;
    float t, z;
    const int32_t jx = (int32_t)glm_f2u(x);
    const int32_t ix = jx & 0x7fffffff;
    if (ix >= 0x7f800000) {
        if (jx >= 0) return one / x + one;
        return one / x - one;
    }
    if (ix < 0x41b00000) {            // |x| < 22
        if (ix == 0) return x;
        if (ix < 0x24000000) return x * (one + x);  // |x| < 2^-55
        const float ax = glm_u2f((uint32_t)ix);
        if (ix >= 0x3f800000) {
            t = glm_expm1f(two * ax);
            z = one - two / (t + two);
        } else {
            t = glm_expm1f(-two * ax);
            z = -t / (t + two);
        }
    } else {
        z = one - tiny;
    }
    return (jx >= 0) ? z : -z;
}

// bits of 2^(i/32) minus i << 47, so that adding k << 47 for k = 32 q + i yields 2^(k/32)
#define GLM_EXP2_TAB                                                                                                 \
    {                                                                                                                \
        0x3ff0000000000000ull, 0x3fefd9b0d3158574ull, 0x3fefb5586cf9890full, 0x3fef9301d0125b51ull,                  \
        0x3fef72b83c7d517bull, 0x3fef54873168b9aaull, 0x3fef387a6e756238ull, 0x3fef1e9df51fdee1ull,                  \
        0x3fef06fe0a31b715ull, 0x3feef1a7373aa9cbull, 0x3feedea64c123422ull, 0x3feece086061892dull,                  \
        0x3feebfdad5362a27ull, 0x3feeb42b569d4f82ull, 0x3feeab07dd485429ull, 0x3feea47eb03a5585ull,                  \
        0x3feea09e667f3bcdull, 0x3fee9f75e8ec5f74ull, 0x3feea11473eb0187ull, 0x3feea589994cce13ull,                  \
        0x3feeace5422aa0dbull, 0x3feeb737b0cdc5e5ull, 0x3feec49182a3f090ull, 0x3feed503b23e255dull,                  \
        0x3feee89f995ad3adull, 0x3feeff76f2fb5e47ull, 0x3fef199bdd85529cull, 0x3fef3720dcef9069ull,                  \
        0x3fef5818dcfba487ull, 0x3fef7c97337b9b5full, 0x3fefa4afa2a490daull, 0x3fefd0765b6e4540ull                   \
    }

// T: the 32 table entries above, wherever the caller keeps them (a kernel may hold them in LDS)
GLM_FN float glm_expf_tab(float x, const uint64_t* T)
{
    const double C0 = 0x1.c6af84b912394p-5 / 32 / 32 / 32, C1 = 0x1.ebfce50fac4f3p-3 / 32 / 32,
                 C2 = 0x1.62e42ff0c52d6p-1 / 32;
    const double InvLn2N = 0x1.71547652b82fep+0 * 32, Shift = 0x1.8p+52;
    const double xd = (double)x;
    const uint32_t abstop = (glm_f2u(x) >> 20) & 0x7ff;
    if (abstop >= 0x42b) {            // |x| >= 88 or NaN
        if (glm_f2u(x) == 0xff800000u) return 0.0f;
        if (abstop >= 0x7f8) return x + x;
        if (x > 0x1.62e42ep6f) return glm_u2f(0x7f800000u);
        if (x < -0x1.9fe368p6f) return 0.0f;
    }
    double kd = __builtin_fma(InvLn2N, xd, Shift);
    const uint64_t ki = glm_d2u(kd);
    kd -= Shift;
    const double r = __builtin_fma(InvLn2N, xd, -kd);
    const double s = glm_u2d(T[ki % 32] + (ki << 47));
    const double p = __builtin_fma(C0, r, C1);
    const double r2 = r * r;
    double y = __builtin_fma(C2, r, 1.0);
    y = __builtin_fma(p, r2, y);
    y = y * s;
    return (float)y;
}

GLM_FN float glm_expf(float x)
{
    const uint64_t T[32] = GLM_EXP2_TAB;
    return glm_expf_tab(x, T);
}

GLM_FN float glm_logf(float x)
{
    const double invc[16] = {0x1.661ec79f8f3bep+0, 0x1.571ed4aaf883dp+0, 0x1.49539f0f010bp+0,  0x1.3c995b0b80385p+0,
                             0x1.30d190c8864a5p+0, 0x1.25e227b0b8eap+0,  0x1.1bb4a4a1a343fp+0, 0x1.12358f08ae5bap+0,
                             0x1.0953f419900a7p+0, 0x1p+0,               0x1.e608cfd9a47acp-1, 0x1.ca4b31f026aap-1,
                             0x1.b2036576afce6p-1, 0x1.9c2d163a1aa2dp-1, 0x1.886e6037841edp-1, 0x1.767dcf5534862p-1};
    const double logc[16] = {-0x1.57bf7808caadep-2, -0x1.2bef0a7c06ddbp-2, -0x1.01eae7f513a67p-2, -0x1.b31d8a68224e9p-3,
                             -0x1.6574f0ac07758p-3, -0x1.1aa2bc79c81p-3,   -0x1.a4e76ce8c0e5ep-4, -0x1.1973c5a611cccp-4,
                             -0x1.252f438e10c1ep-5, 0x0p+0,                0x1.aa5aa5df25984p-5,  0x1.c5e53aa362eb4p-4,
                             0x1.526e57720db08p-3,  0x1.bc2860d22477p-3,   0x1.1058bc8a07ee1p-2,  0x1.4043057b6ee09p-2};
    const double Ln2 = 0x1.62e42fefa39efp-1;
    const double A0 = -0x1.00ea348b88334p-2, A1 = 0x1.5575b0be00b6ap-2, A2 = -0x1.ffffef20a4123p-2;
    uint32_t ix = glm_f2u(x);
    if (ix == 0x3f800000u) return 0.0f;
    if (ix - 0x00800000u >= 0x7f800000u - 0x00800000u) {  // x < 2^-126, inf or NaN
        if (ix * 2 == 0) return glm_u2f(0xff800000u);
        if (ix == 0x7f800000u) return x;
        if ((ix & 0x80000000u) || ix * 2 >= 0xff000000u) return glm_u2f(0x7fc00000u);
        ix = glm_f2u(x * 0x1p23f);
        ix -= 23u << 23;
    }
    const uint32_t tmp = ix - 0x3f330000u;
    const int i = (int)((tmp >> 19) % 16);
    const int k = (int32_t)tmp >> 23;
    const uint32_t iz = ix - (tmp & 0xff800000u);
    const double z = (double)glm_u2f(iz);
    const double r = __builtin_fma(z, invc[i], -1.0);
    const double y0 = __builtin_fma((double)k, Ln2, logc[i]);
    const double r2 = r * r;
    double y = __builtin_fma(A1, r, A2);
    y = __builtin_fma(A0, r2, y);
    y = __builtin_fma(y, r2, y0 + r);
    return (float)y;
}
