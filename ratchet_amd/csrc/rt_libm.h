// The libm-level routines of the kernels, in portable C++ so that the same text can be compiled for the host and checked
// against the C library there (tests/device_math_check.cpp does, with g++): the includer defines
//   RT_FN     the function qualifiers (`__device__ inline` in the kernels, `static inline` on the host)
//   RT_TABLE  the qualifiers of a constant table (`__device__ static const` / `static const`)
//
// The libm routines of the unary ops are restated operation by operation so that their float32 results equal, bit for
// bit, what the x86-64 glibc 2.35 `tanhf`, `expf`, `logf`, `sinf` and `cosf` return (checked on the CPU over all 2^32
// inputs with this same code compiled by g++).  ratchet's CPU executor calls exactly those through Rust's f32::tanh /
// f32::exp / f32::ln / f32::sin / f32::cos (crates/ratchet-core/src/cpu/unary.rs:46-65, cpu/softmax.rs:30, cpu/rope.rs), and GELU's `1 + tanh(..)` cancellation turns a
// 1-ulp tanh difference into hundreds of ulps, so "close" is not good enough there.
//   tanhf/expm1f: the classic fdlibm float algorithms (float arithmetic only).
//   expf: the table-driven double-precision algorithm (2^(k/32) table, degree-3 polynomial), with the
//         reduction r = fma(InvLn2N, x, -kd) that an FMA build of the routine performs.
//   logf: a 16-entry table of (1/c, log c) and a cubic, in double.  sinf / cosf: the quadrant and the reduced argument in
//         double (x - n * pi/2 as one fma, as an FMA build performs it), sine and cosine polynomials in double.
// Everything here must be compiled with -ffp-contract=off: each float operation below is meant to round on its own.
//
// Provenance.  The routines below are restatements of published algorithms, with their published constants (a result
// that must equal the C library's bit for bit cannot use others); no file of either library was copied.
//   rt_expm1f, rt_tanhf: the float versions of FreeBSD's msun / Sun's fdlibm `s_expm1f.c` and `s_tanhf.c`, as glibc
//     ships them.  fdlibm's notice, which asks to be kept with the algorithm:
//       Copyright (C) 1993 by Sun Microsystems, Inc. All rights reserved.
//       Developed at SunPro, a Sun Microsystems, Inc. business.
//       Permission to use, copy, modify, and distribute this software is freely granted, provided that this notice
//       is preserved.
//   rt_expf: the single-precision exp of Arm's optimized-routines (`math/expf.c`, `math/exp2f_data.c`; Copyright (c)
//     2017-2018 Arm Limited, SPDX-License-Identifier: MIT), which glibc 2.27 and later use for `expf`: the 32-entry
//     table follows from its defining formula (the comment above it), the three polynomial coefficients and the
//     reduction constants are the published ones.
//   rt_logf, rt_sinf, rt_cosf: the single-precision log, sin and cos of the same Arm optimized-routines (`math/logf.c`,
//     `math/logf_data.c`, `math/sinf.c`, `math/cosf.c`, `math/sincosf.h`, `math/sincosf_data.c`; Copyright (c) 2017-2018 Arm
//     Limited, SPDX-License-Identifier: MIT), which glibc uses for `logf`, `sinf` and `cosf`: the tables and coefficients are
//     the published ones.
#ifndef RT_LIBM_H
#define RT_LIBM_H

#include <math.h>
#include <stdint.h>

RT_FN uint32_t f2u(float f) { return __builtin_bit_cast(uint32_t, f); }
RT_FN float u2f(uint32_t u) { return __builtin_bit_cast(float, u); }

// ---- expm1f, fdlibm -------------------------------------------------------------------------------------
RT_FN float rt_expm1f(float x) {
    const float one = 1.0f, huge = 1.0e+30f, tiny = 1.0e-30f;
    const float o_threshold = 8.8721679688e+01f, ln2_hi = 6.9313812256e-01f, ln2_lo = 9.0580006145e-06f,
                invln2 = 1.4426950216e+00f;
    const float Q1 = -3.3333335072e-02f, Q2 = 1.5873016091e-03f, Q3 = -7.9365076090e-05f, Q4 = 4.0082177293e-06f,
                Q5 = -2.0109921195e-07f;
    float y, hi, lo, c = 0.0f, t, e, hxs, hfx, r1;
    int32_t k;
    uint32_t hx = f2u(x);
    const uint32_t xsb = hx & 0x80000000u;
    hx &= 0x7fffffffu;
    if (hx >= 0x4195b844u) {                       // |x| >= 27 ln2
        if (hx >= 0x42b17218u) {                   // |x| >= 88.72
            if (hx > 0x7f800000u) return x + x;    // NaN
            if (hx == 0x7f800000u) return xsb == 0 ? x : -1.0f;
            if (x > o_threshold) return huge * huge;
        }
        if (xsb != 0) {
            if (x + tiny < 0.0f) return tiny - one;
        }
    }
    if (hx > 0x3eb17218u) {                        // |x| > 0.5 ln2
        if (hx < 0x3F851592u) {                    // |x| < 1.5 ln2
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
    } else if (hx < 0x33000000u) {                 // |x| < 2^-25
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
        y = u2f(f2u(y) + ((uint32_t)k << 23));
        return y - one;
    }
    if (k < 23) {
        t = u2f(0x3f800000u - (0x1000000u >> k));  // 1 - 2^-k
        y = t - (e - x);
        y = u2f(f2u(y) + ((uint32_t)k << 23));
    } else {
        t = u2f((uint32_t)(0x7f - k) << 23);       // 2^-k
        y = x - (e + t);
        y += one;
        y = u2f(f2u(y) + ((uint32_t)k << 23));
    }
    return y;
}

// ---- tanhf, fdlibm --------------------------------------------------------------------------------------
// fdlibm's tanhf calls expm1f on 2|x| (|x| >= 1) or -2|x| (|x| < 1) and divides once more.  The same operations in the
// same order, laid out without branches: every lane of a wave evaluates one argument reduction, one polynomial and the
// few endings that these arguments can reach (k = 0, -1, <= -2 for the negative arguments, k >= 3 for the positive ones;
// expm1f's k = 1 ending cannot occur), and selects.  With branches a wave whose lanes disagree ran every ending in turn
// behind scalar branch code (137 vector and 114 scalar instructions per GELU element; now 116 and 9: f32 GELU on 2^26
// elements 2.36 -> 3.53 TB/s, tanh 2.71 -> 3.33).
RT_FN float rt_tanhf(float x) {
    const float one = 1.0f, two = 2.0f;
    const float ln2_hi = 6.9313812256e-01f, ln2_lo = 9.0580006145e-06f, invln2 = 1.4426950216e+00f;
    const float Q1 = -3.3333335072e-02f, Q2 = 1.5873016091e-03f, Q3 = -7.9365076090e-05f, Q4 = 4.0082177293e-06f,
                Q5 = -2.0109921195e-07f;
    const uint32_t ux = f2u(x), ix = ux & 0x7fffffffu;
    const float ax = u2f(ix);
    const bool big = ix >= 0x3f800000u;                        // |x| >= 1
    const float a = big ? two * ax : -two * ax;                // expm1f's argument, |a| < 44 where the result is used
    // expm1f(a): argument reduction a = k ln2 + r
    const uint32_t ha = f2u(a) & 0x7fffffffu;
    int32_t k = (int32_t)(invln2 * a + (big ? 0.5f : -0.5f));
    k = ha < 0x3F851592u ? (big ? 1 : -1) : k;                 // |a| < 1.5 ln2
    k = ha <= 0x3eb17218u ? 0 : k;                             // |a| <= 0.5 ln2: no reduction (t = 0 below leaves a as it is)
    const float t = (float)k;
    const float hi = a - t * ln2_hi;
    const float lo = t * ln2_lo;
    const float r = hi - lo;
    const float c = (hi - r) - lo;
    const float hfx = 0.5f * r;
    const float hxs = r * hfx;
    const float r1 = one + hxs * (Q1 + hxs * (Q2 + hxs * (Q3 + hxs * (Q4 + hxs * Q5))));
    const float tt = 3.0f - r1 * hfx;
    const float e0 = hxs * ((r1 - tt) / (6.0f - r * tt));
    const float v0 = r - (r * e0 - hxs);                       // k == 0
    const float e = (r * (e0 - c) - c) - hxs;
    const float vm1 = 0.5f * (r - e) - 0.5f;                   // k == -1
    // k <= -2 and k > 56: 1 - (e - r), scaled by 2^k, minus one; 2 <= k < 23: (1 - 2^-k) - (e - r), scaled
    const bool mid = k >= 2 && k < 23;
    const uint32_t kbits = (uint32_t)k << 23;
    float y = (mid ? u2f(0x3f800000u - (0x1000000u >> (k & 31))) : one) - (e - r);
    y = u2f(f2u(y) + kbits);
    y = mid ? y : y - one;
    // 23 <= k <= 56: r - (e + 2^-k) + 1, scaled
    float y2 = r - (e + u2f((uint32_t)(0x7f - k) << 23));
    y2 += one;
    y2 = u2f(f2u(y2) + kbits);
    float em1 = (k >= 23 && k <= 56) ? y2 : y;
    em1 = k == -1 ? vm1 : em1;
    em1 = k == 0 ? v0 : em1;
    em1 = ha < 0x33000000u ? a : em1;                          // |a| < 2^-25: expm1f returns its argument
    // tanh: |x| >= 1: 1 - 2 / (em1 + 2); |x| < 1: -em1 / (em1 + 2)
    const float q = (big ? two : -em1) / (em1 + two);
    float z = big ? one - q : q;
    z = ix >= 0x41b00000u ? one : z;                           // |x| >= 22 (and infinity): 1 - tiny rounds to 1
    z = (ux >> 31) ? -z : z;
    z = ix < 0x24000000u ? x : z;                              // |x| < 2^-55 (and zero): x * (1 + x) is x
    z = x != x ? x + x : z;                                    // NaN
    return z;
}

// ---- expf, table-driven double algorithm ----------------------------------------------------------------
// T[i] = bits(2^(i/32)) - (i << 47)
RT_TABLE uint64_t rt_exp2f_tab[32] = {
    0x3ff0000000000000ull, 0x3fefd9b0d3158574ull, 0x3fefb5586cf9890full, 0x3fef9301d0125b51ull,
    0x3fef72b83c7d517bull, 0x3fef54873168b9aaull, 0x3fef387a6e756238ull, 0x3fef1e9df51fdee1ull,
    0x3fef06fe0a31b715ull, 0x3feef1a7373aa9cbull, 0x3feedea64c123422ull, 0x3feece086061892dull,
    0x3feebfdad5362a27ull, 0x3feeb42b569d4f82ull, 0x3feeab07dd485429ull, 0x3feea47eb03a5585ull,
    0x3feea09e667f3bcdull, 0x3fee9f75e8ec5f74ull, 0x3feea11473eb0187ull, 0x3feea589994cce13ull,
    0x3feeace5422aa0dbull, 0x3feeb737b0cdc5e5ull, 0x3feec49182a3f090ull, 0x3feed503b23e255dull,
    0x3feee89f995ad3adull, 0x3feeff76f2fb5e47ull, 0x3fef199bdd85529cull, 0x3fef3720dcef9069ull,
    0x3fef5818dcfba487ull, 0x3fef7c97337b9b5full, 0x3fefa4afa2a490daull, 0x3fefd0765b6e4540ull};

// tab: rt_exp2f_tab or a copy of it (a kernel that evaluates many exponentials stages the 256 bytes in LDS: 64 lanes that
// gather from it cost less there than through the vector memory path; f32 exp on 2^26 elements 5.6 -> 6.35 TB/s)
RT_FN float rt_expf_tab(float x, const uint64_t* tab) {
    const double N = 32.0;
    const double InvLn2N = 0x1.71547652b82fep+0 * N;
    const double SHIFT = 0x1.8p52;
    const double C0 = 0x1.c6af84b912394p-5 / N / N / N, C1 = 0x1.ebfce50fac4f3p-3 / N / N, C2 = 0x1.62e42ff0c52d6p-1 / N;
    // The evaluation runs for every input and the special cases are selected afterwards, all without a branch: the table
    // loads of the elements a thread holds are then issued together instead of each behind its own range test (f32 exp on
    // 2^26 elements: 4.5 -> 5.6 TB/s).  Inputs out of range (and NaN) produce some double here, never a trap.
    const double xd = (double)x;
    const double z = InvLn2N * xd;
    double kd = z + SHIFT;
    const uint64_t ki = __builtin_bit_cast(uint64_t, kd);
    kd -= SHIFT;
    const double r = __builtin_fma(InvLn2N, xd, -kd);
    uint64_t t = tab[ki & 31];
    t += ki << (52 - 5);
    const double s = __builtin_bit_cast(double, t);
    const double p = __builtin_fma(C0, r, C1);
    const double r2 = r * r;
    double y = __builtin_fma(C2, r, 1.0);
    y = __builtin_fma(p, r2, y);
    y = y * s;
    float res = (float)y;
    res = x < -0x1.9fe368p6f ? 0.0f : res;                     // underflow, -inf
    res = x > 0x1.62e42ep6f ? __builtin_huge_valf() : res;     // overflow, +inf
    res = x != x ? x + x : res;                                // NaN
    return res;
}

RT_FN float rt_expf(float x) { return rt_expf_tab(x, rt_exp2f_tab); }

// logf as glibc computes it (sysdeps/ieee754/flt-32/e_logf.c, the algorithm of ARM's optimized routines): x = 2^k * z
// with z in [0x1.66p-1, 0x1.66p0), c = the centre of the sixteenth of that interval z lies in, with 1/c and log(c) from
// a table; log(x) = log1p(z/c - 1) + log(c) + k ln 2, a cubic in r = z/c - 1, all in double, rounded once.  Without a
// branch: the evaluation runs for every input (a subnormal one scaled by 2^23 first) and the special cases are
// selected afterwards.  Equal to this machine's logf on all 2^32 inputs (tests/device_math_check.cpp).
RT_TABLE double rt_logf_tab[32] = {
    0x1.661ec79f8f3bep+0, -0x1.57bf7808caadep-2, 0x1.571ed4aaf883dp+0, -0x1.2bef0a7c06ddbp-2, 0x1.49539f0f010bp+0,  -0x1.01eae7f513a67p-2,
    0x1.3c995b0b80385p+0, -0x1.b31d8a68224e9p-3, 0x1.30d190c8864a5p+0, -0x1.6574f0ac07758p-3, 0x1.25e227b0b8eap+0,  -0x1.1aa2bc79c81p-3,
    0x1.1bb4a4a1a343fp+0, -0x1.a4e76ce8c0e5ep-4, 0x1.12358f08ae5bap+0, -0x1.1973c5a611cccp-4, 0x1.0953f419900a7p+0, -0x1.252f438e10c1ep-5,
    0x1p+0,               0x0p+0,                0x1.e608cfd9a47acp-1, 0x1.aa5aa5df25984p-5,  0x1.ca4b31f026aap-1,  0x1.c5e53aa362eb4p-4,
    0x1.b2036576afce6p-1, 0x1.526e57720db08p-3,  0x1.9c2d163a1aa2dp-1, 0x1.bc2860d22477p-3,   0x1.886e6037841edp-1, 0x1.1058bc8a07ee1p-2,
    0x1.767dcf5534862p-1, 0x1.4043057b6ee09p-2,
};

RT_FN float rt_logf_tab_at(float x, const double* tab) {
    const double A0 = -0x1.00ea348b88334p-2, A1 = 0x1.5575b0be00b6ap-2, A2 = -0x1.ffffef20a4123p-2, LN2 = 0x1.62e42fefa39efp-1;
    uint32_t ix = f2u(x);
    const bool sub = ix < 0x00800000u;                        // subnormal (or zero, replaced below): scaled up by 2^23
    const uint32_t scaled = f2u(x * 0x1p23f) - (23u << 23);
    uint32_t iw = sub ? scaled : ix;
    const uint32_t tmp = iw - 0x3f330000u;
    const uint32_t i = (tmp >> 19) & 15u;
    const int32_t k = (int32_t)tmp >> 23;                     // arithmetic shift
    const uint32_t iz = iw - (tmp & 0xff800000u);
    const double invc = tab[2 * i], logc = tab[2 * i + 1];
    const double z = (double)u2f(iz);
    const double r = z * invc - 1.0;
    const double y0 = logc + (double)k * LN2;
    const double r2 = r * r;
    double y = A1 * r + A2;
    y = A0 * r2 + y;
    y = y * r2 + (y0 + r);
    float res = (float)y;
    res = ix == 0x3f800000u ? 0.0f : res;                     // log(1) = +0 exactly
    res = ix == 0x7f800000u ? x : res;                        // +inf
    res = (ix & 0x80000000u) != 0 || ix > 0x7f800000u ? (x - x) / 0.0f : res;      // negative or NaN: NaN
    res = (ix << 1) == 0 ? -__builtin_huge_valf() : res;      // +-0: -inf
    return res;
}

RT_FN float rt_logf(float x) { return rt_logf_tab_at(x, rt_logf_tab); }
// sinf / cosf as glibc computes them (sysdeps/ieee754/flt-32/s_sinf.c, s_cosf.c, s_sincosf.h: the algorithm of ARM's
// optimized routines): the argument reduced to [-pi/4, pi/4] in double (one multiply and a rounded quadrant below 120,
// a 192-bit slice of 4/pi above), a degree-7 sine or degree-8 cosine polynomial in double picked by the quadrant, one
// rounding to float.
RT_TABLE uint32_t rt_inv_pio4[24] = {0xa2,       0xa2f9,     0xa2f983,   0xa2f9836e, 0xf9836e4e, 0x836e4e44, 0x6e4e4415, 0x4e441529,
                                     0x441529fc, 0x1529fc27, 0x29fc2757, 0xfc2757d1, 0x2757d1f5, 0x57d1f534, 0xd1f534dd, 0xf534ddc0,
                                     0x34ddc0db, 0xddc0db62, 0xc0db6295, 0xdb629599, 0x6295993c, 0x95993c43, 0x993c4390, 0x3c439041};

// the polynomial of quadrant n on the reduced x (x2 = x * x): sine for even n, cosine for odd n; neg: quadrants 2 and 3,
// whose cosine coefficients carry the other sign (the same as negating the value: every step is symmetric in the sign).
// Both are evaluated and one is selected: the lanes of a wave lie in different quadrants.
RT_FN float rt_sincosf_poly(double x, double x2, int n, bool neg) {
    const double S1 = -0x1.555545995a603p-3, S2 = 0x1.1107605230bc4p-7, S3 = -0x1.994eb3774cf24p-13;
    const double C0 = 0x1p0, C1 = -0x1.ffffffd0c621cp-2, C2 = 0x1.55553e1068f19p-5, C3 = -0x1.6c087e89a359dp-10, C4 = 0x1.99343027bf8c3p-16;
    const double x3 = x * x2;
    const double s1 = S2 + x2 * S3;
    const double x7 = x3 * x2;
    const double s = x + x3 * S1;
    const double sinv = s + x7 * s1;
    const double x4 = x2 * x2;
    const double c2 = C3 + x2 * C4;
    const double c1 = C0 + x2 * C1;
    const double x6 = x4 * x2;
    const double c = c1 + x4 * C2;
    const double cosv = c + x6 * c2;
    return (float)((n & 1) ? (neg ? -cosv : cosv) : sinv);
}

// COS: 0 sine, 1 cosine.  The reduction below 120 runs for every input (with 0 in place of larger ones) and covers
// |y| < pi/4 too (quadrant 0, x unchanged); only the slice-of-4/pi reduction of larger arguments sits behind a branch.
template <int COS> RT_FN float rt_sincosf(float y) {
    const uint32_t xi = f2u(y);
    const uint32_t top = (xi >> 20) & 0x7ffu;
    const bool large = top >= 0x42fu;                         // |y| >= 120, inf, NaN
    double x = large ? 0.0 : (double)y;
    const double r = x * 0x1.45F306DC9C883p+23;               // quadrant from x * (2/pi) * 2^24, rounded
    int n = ((int32_t)r + 0x800000) >> 24;
    x = __builtin_fma(-(double)n, 0x1.921FB54442D18p0, x);     // one rounding, as the C library's build for FMA hardware does it
    int sign = 0;
    if (large && top < 0x7f8u) {
        const uint32_t* arr = &rt_inv_pio4[(xi >> 26) & 15];
        const int shift = (int)((xi >> 23) & 7);
        uint32_t m = (xi & 0xffffffu) | 0x800000u;
        m <<= shift;
        uint64_t res0 = (uint64_t)(uint32_t)(m * arr[0]);
        const uint64_t res1 = (uint64_t)m * arr[4];
        const uint64_t res2 = (uint64_t)m * arr[8];
        res0 = (res2 >> 32) | (res0 << 32);
        res0 += res1;
        const uint64_t q = (res0 + (1ull << 61)) >> 62;
        res0 -= q << 62;
        x = (double)(int64_t)res0 * 0x1.921FB54442D18p-62;
        n = (int)q;
        sign = (int)(xi >> 31);
    }
    const int ns = n + sign;
    const double s = ((ns & 3) == 1 || (ns & 3) == 2) ? -1.0 : 1.0;          // sign of sine in quadrants 0..3: + - - +
    float res = rt_sincosf_poly(x * s, x * x, n ^ COS, (ns & 2) != 0);
    res = top < 0x398u ? (COS ? 1.0f : y) : res;              // |y| < 2^-12
    res = top >= 0x7f8u ? (y - y) / 0.0f : res;               // inf, NaN
    return res;
}

RT_FN float rt_sinf(float x) { return rt_sincosf<0>(x); }
RT_FN float rt_cosf(float x) { return rt_sincosf<1>(x); }

// bf16 <-> f32 with the rounding of half::bf16::from_f32 (round to nearest even, NaN quieted)
RT_FN float bf2f(uint16_t b) { return u2f((uint32_t)b << 16); }
RT_FN uint16_t f2bf(float f) {
    const uint32_t x = f2u(f);
    if ((x & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((x >> 16) | 0x0040u);
    const uint32_t round_bit = 0x00008000u;
    if ((x & round_bit) != 0 && (x & (3u * round_bit - 1u)) != 0) return (uint16_t)((x >> 16) + 1);
    return (uint16_t)(x >> 16);
}

#endif
