// tanh and expm1 for f64 values the way the host's C library computes them, so that tanh and gelu_tanh of F64
// tensors get the CPU's bits (ref: src/backend/cpu/mod.rs:378-403: f64::tanh, that is libm's). glibc's tanh and
// expm1 are fdlibm's (s_tanh.c, s_expm1.c; the polynomial of expm1 in the split form glibc evaluates it in),
// straight-line f64 arithmetic, restated here step for step like their f32 versions in f32_like_libm.hpp. No walk
// over all inputs is possible in f64: compiled for the host and compared with the library's (tests/libm_check.cpp),
// neither differs for any of 480 million sampled inputs (arbitrary bits, (-25, 25), (-2, 2), and every binade down
// to 2^-70); with the polynomial in Horner form 69 078 of them differ, which is what tells the two forms apart.
//
// The algorithms and constants are fdlibm's, whose notice reads: "Copyright (C) 1993 by Sun Microsystems, Inc. All
// rights reserved. Developed at SunPro, a Sun Microsystems, Inc. business. Permission to use, copy, modify, and
// distribute this software is freely granted, provided that this notice is preserved."
#pragma once
#include <cstdint>
#include <cstring>

namespace hmr {

__host__ __device__ inline uint64_t libm_bits64(double x) {
    uint64_t b;
    memcpy(&b, &x, 8);
    return b;
}
__host__ __device__ inline double libm_double(uint64_t b) {
    double x;
    memcpy(&x, &b, 8);
    return x;
}
__host__ __device__ inline uint32_t libm_high(double x) { return (uint32_t)(libm_bits64(x) >> 32); }
__host__ __device__ inline double libm_scale(double y, int k) { return libm_double(libm_bits64(y) + ((uint64_t)(uint32_t)(k << 20) << 32)); }
__host__ __device__ inline double expm1_like_libm(double x) {
    const double one = 1.0, huge = 1.0e+300, tiny = 1.0e-300, o_threshold = 7.09782712893383973096e+02,
                 ln2_hi = 6.93147180369123816490e-01, ln2_lo = 1.90821492927058770002e-10, invln2 = 1.44269504088896338700e+00;
    const double Q1 = -3.33333333333331316428e-02, Q2 = 1.58730158725481460165e-03, Q3 = -7.93650757867487942473e-05,
                 Q4 = 4.00821782732936239552e-06, Q5 = -2.01099218183624371326e-07;
    double y, hi, lo, c = 0.0, t, e, hxs, hfx, r1;
    int32_t k;
    uint32_t hx = libm_high(x);
    const uint32_t xsb = hx & 0x80000000u;
    hx &= 0x7fffffffu;
    if (hx >= 0x4043687Au) {
        if (hx >= 0x40862E42u) {
            if (hx >= 0x7ff00000u) {
                if (((hx & 0xfffff) | (uint32_t)libm_bits64(x)) != 0) return x + x;
                return xsb == 0 ? x : -1.0;
            }
            if (x > o_threshold) return huge * huge;
        }
        if (xsb != 0) return tiny - one;
    }
    if (hx > 0x3fd62e42u) {
        if (hx < 0x3FF0A2B2u) {
            if (xsb == 0) { hi = x - ln2_hi; lo = ln2_lo; k = 1; }
            else { hi = x + ln2_hi; lo = -ln2_lo; k = -1; }
        } else {
            k = (int32_t)(invln2 * x + (xsb == 0 ? 0.5 : -0.5));
            t = k;
            hi = x - t * ln2_hi;
            lo = t * ln2_lo;
        }
        x = hi - lo;
        c = (hi - x) - lo;
    } else if (hx < 0x3c900000u) {
        t = huge + x;
        return x - (t - (huge + x));
    } else {
        k = 0;
    }
    hfx = 0.5 * x;
    hxs = x * hfx;
    const double R1 = one + hxs * Q1, h2 = hxs * hxs, R2 = Q2 + hxs * Q3, h4 = h2 * h2, R3 = Q4 + hxs * Q5;
    r1 = R1 + h2 * R2 + h4 * R3;
    t = 3.0 - r1 * hfx;
    e = hxs * ((r1 - t) / (6.0 - x * t));
    if (k == 0) return x - (x * e - hxs);
    e = (x * (e - c) - c);
    e -= hxs;
    if (k == -1) return 0.5 * (x - e) - 0.5;
    if (k == 1) {
        if (x < -0.25) return -2.0 * (e - (x + 0.5));
        return one + 2.0 * (x - e);
    }
    if (k <= -2 || k > 56) {
        y = one - (e - x);
        y = libm_scale(y, k);
        return y - one;
    }
    if (k < 20) {
        t = libm_double((uint64_t)(0x3ff00000u - (0x200000u >> k)) << 32);
        y = t - (e - x);
        y = libm_scale(y, k);
    } else {
        t = libm_double((uint64_t)((uint32_t)(0x3ff - k) << 20) << 32);
        y = x - (e + t);
        y += one;
        y = libm_scale(y, k);
    }
    return y;
}
__host__ __device__ inline double tanh_like_libm(double x) {
    const double one = 1.0, two = 2.0, tiny = 1.0e-300;
    double t, z;
    const uint32_t jx = libm_high(x), ix = jx & 0x7fffffffu, lx = (uint32_t)libm_bits64(x);
    const bool neg = (jx >> 31) != 0;
    if (ix >= 0x7ff00000u) return neg ? one / x - one : one / x + one;
    if (ix < 0x40360000u) {
        if ((ix | lx) == 0) return x;
        if (ix < 0x3c800000u) return x * (one + x);
        const double ax = libm_double(libm_bits64(x) & 0x7fffffffffffffffull);
        if (ix >= 0x3ff00000u) { t = expm1_like_libm(two * ax); z = one - two / (t + two); }
        else { t = expm1_like_libm(-two * ax); z = -t / (t + two); }
    } else {
        z = one - tiny;
    }
    return neg ? -z : z;
}

}  // namespace hmr
