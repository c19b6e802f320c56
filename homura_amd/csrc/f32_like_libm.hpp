// tanh, expm1 and log1p for f32 values the way the host's C library computes tanhf, expm1f and log1pf, so that
// tanh, gelu_tanh and log_sigmoid (ref: src/backend/cpu/mod.rs:378-403: f32::tanh, f32::ln_1p and f32::exp, that
// is libm's) get the CPU's bits. The library's functions are good to an ulp or two, and gelu_tanh's 1 + tanh
// cancels next to its zero: evaluated with correctly rounded functions instead, results lay up to 2, 2 and 178
// ulp from the CPU's. glibc's three routines are the float versions of Sun's fdlibm (s_tanhf.c, s_expm1f.c,
// s_log1pf.c): straight-line f32 arithmetic, restated here step for step from their published algorithms.
//   tanh(x)   = 1 - 2 / (expm1(2|x|) + 2) for |x| >= 1, -t / (t + 2) with t = expm1(-2|x|) below; 1 from 22 on
//   expm1(x)  = x = k ln2 + r (ln2 in two pieces), a rational approximation in r^2 / 2 with five coefficients,
//               and 2^k put back case by case (k = 0, -1, 1, k <= -2 or > 56, k < 23, otherwise)
//   log1p(x)  = k ln2 + log1p(f) with 1 + x = 2^k (1 + f), sqrt(2)/2 < 1 + f < sqrt(2), a correction term for
//               the rounding of 1 + x, and a degree-7 polynomial in s^2, s = f / (2 + f)
// Every step is an IEEE f32 operation (this library compiles without contraction and with correctly rounded
// division), so the same source gives the same bits on the host: tests/libm_check.cpp compares each function
// with the host library's over all 2^32 inputs, and none differs.
//
// The algorithms and constants are fdlibm's, whose notice reads: "Copyright (C) 1993 by Sun Microsystems, Inc. All
// rights reserved. Developed at SunPro, a Sun Microsystems, Inc. business. Permission to use, copy, modify, and
// distribute this software is freely granted, provided that this notice is preserved."
#pragma once
#include <cstdint>
#include <cstring>

namespace hmr {

__host__ __device__ inline uint32_t libm_bits(float x) {
    uint32_t b;
    memcpy(&b, &x, 4);
    return b;
}
__host__ __device__ inline float libm_float(uint32_t b) {
    float x;
    memcpy(&x, &b, 4);
    return x;
}

// expm1f. The library's source branches on k; here the cases are computed side by side and selected, each with the
// library's own operations: lanes of a wave would take different branches anyway, and without them the compiler
// can interleave the independent elements a lane holds (these are chains of some two hundred dependent operations).
__host__ __device__ inline float expm1f_like_libm(float x0) {
    const float one = 1.0f, tiny = 1.0e-30f, huge = 1.0e+30f;
    const float o_threshold = 8.8721679688e+01f, ln2_hi = 6.9313812256e-01f, ln2_lo = 9.0580006145e-06f, invln2 = 1.4426950216e+00f;
    const float Q1 = -3.3333335072e-02f, Q2 = 1.5873016091e-03f, Q3 = -7.9365076090e-05f, Q4 = 4.0082177293e-06f, Q5 = -2.0109921195e-07f;
    const uint32_t bits = libm_bits(x0), hx = bits & 0x7fffffffu;
    const bool neg = (bits >> 31) != 0;
    // argument reduction
    const bool reduce = hx > 0x3eb17218u, unit = hx < 0x3F851592u;
    const int32_t kg = static_cast<int32_t>(invln2 * x0 + (neg ? -0.5f : 0.5f));
    const int32_t k = reduce ? (unit ? (neg ? -1 : 1) : kg) : 0;
    const float t0 = static_cast<float>(k);
    const float hi = x0 - t0 * ln2_hi, lo = t0 * ln2_lo;
    const float xr = hi - lo;
    const float x = reduce ? xr : x0;
    const float c = reduce ? (hi - xr) - lo : 0.0f;
    // primary range
    const float hfx = 0.5f * x, hxs = x * hfx;
    const float r1 = one + hxs * (Q1 + hxs * (Q2 + hxs * (Q3 + hxs * (Q4 + hxs * Q5))));
    const float t = 3.0f - r1 * hfx;
    const float e0 = hxs * ((r1 - t) / (6.0f - x * t));
    const float res_k0 = x - (x * e0 - hxs);
    float e = (x * (e0 - c) - c);
    e -= hxs;
    const float res_m1 = 0.5f * (x - e) - 0.5f;
    const float res_p1 = x < -0.25f ? -2.0f * (e - (x + 0.5f)) : one + 2.0f * (x - e);
    const uint32_t kshift = static_cast<uint32_t>(k) << 23;
    const float ya = one - (e - x);
    const float res_far = libm_float(libm_bits(ya) + kshift) - one;
    const uint32_t ks = static_cast<uint32_t>(k) & 31u;  // shifts below are only used for 0 <= k < 23
    const float tb = libm_float(0x3f800000u - (0x1000000u >> ks));
    const float res_lo = libm_float(libm_bits(tb - (e - x)) + kshift);
    const float tc = libm_float(static_cast<uint32_t>(0x7f - k) << 23);
    float yc = x - (e + tc);
    yc += one;
    const float res_hi = libm_float(libm_bits(yc) + kshift);
    float r = k == 0 ? res_k0 : k == -1 ? res_m1 : k == 1 ? res_p1 : (k <= -2 || k > 56) ? res_far : k < 23 ? res_lo : res_hi;
    // |x| < 2^-25
    const float tt = huge + x0;
    r = (!reduce && hx < 0x33000000u) ? x0 - (tt - (huge + x0)) : r;
    // huge and non-finite arguments
    if (hx >= 0x4195b844u) {
        if (hx >= 0x42b17218u) {
            if (hx > 0x7f800000u) return x0 + x0;
            if (hx == 0x7f800000u) return neg ? -1.0f : x0;
            if (x0 > o_threshold) return huge * huge;
        }
        if (neg) return tiny - one;
    }
    return r;
}
__host__ __device__ inline float tanhf_like_libm(float x) {
    const float one = 1.0f, two = 2.0f, tiny = 1.0e-30f;
    const uint32_t jx = libm_bits(x), ix = jx & 0x7fffffffu;
    const bool neg = (jx >> 31) != 0;
    const float ax = libm_float(ix);
    const bool big = ix >= 0x3f800000u;
    const float t = expm1f_like_libm(big ? two * ax : -two * ax);
    const float q = (big ? two : t) / (t + two);
    float z = big ? one - q : -q;
    z = ix < 0x41b00000u ? z : one - tiny;
    float r = neg ? -z : z;
    r = ix < 0x24000000u ? x * (one + x) : r;
    r = ix == 0 ? x : r;
    if (ix >= 0x7f800000u) return neg ? one / x - one : one / x + one;
    return r;
}

// log1pf, its cases side by side like expm1f's (the rare ones, which return early, first).
__host__ __device__ inline float log1pf_like_libm(float x) {
    const float ln2_hi = 6.9313812256e-01f, ln2_lo = 9.0580006145e-06f, two25 = 3.355443200e+07f, zero = 0.0f;
    const float Lp1 = 6.6666668653e-01f, Lp2 = 4.0000000596e-01f, Lp3 = 2.8571429849e-01f, Lp4 = 2.2222198546e-01f,
                Lp5 = 1.8183572590e-01f, Lp6 = 1.5313838422e-01f, Lp7 = 1.4798198640e-01f;
    const int32_t hx = static_cast<int32_t>(libm_bits(x)), ax = hx & 0x7fffffff;
    // the rare cases first
    if (hx < 0x3ed413d7) {
        if (ax >= 0x3f800000) {
            if (x == -1.0f) return -two25 / zero;
            return (x - x) / (x - x);
        }
        if (ax < 0x31000000) {
            if (ax < 0x24800000) return x;
            return x - x * x * 0.5f;
        }
    }
    if (hx >= 0x7f800000) return x + x;
    // -0.2929 < x < 0.41422: no scaling
    const bool direct = hx < 0x3ed413d7 && (hx > 0 || hx <= static_cast<int32_t>(0xbe95f61fu));
    // otherwise 1 + x = 2^k u with a correction c for the rounding of 1 + x
    const bool small = hx < 0x5a000000;
    const float u0 = small ? 1.0f + x : x;
    int32_t hu = static_cast<int32_t>(libm_bits(u0));
    int32_t k = (hu >> 23) - 127;
    float c = small ? ((k > 0) ? 1.0f - (u0 - x) : x - (u0 - 1.0f)) / u0 : 0.0f;
    hu &= 0x007fffff;
    const bool low = hu < 0x3504f7;
    const float u = libm_float(static_cast<uint32_t>(hu) | (low ? 0x3f800000u : 0x3f000000u));
    k = low ? k : k + 1;
    hu = low ? hu : (0x00800000 - hu) >> 2;
    float f = u - 1.0f;
    // the direct case overrides
    f = direct ? x : f;
    k = direct ? 0 : k;
    hu = direct ? 1 : hu;
    c = direct ? 0.0f : c;
    const float fk = static_cast<float>(k);
    const float hfsq = 0.5f * f * f;
    // |f| < 2^-20
    const float Rs = hfsq * (1.0f - 0.66666666666666666f * f);
    const float near_zero = k == 0 ? zero : fk * ln2_hi + (c + fk * ln2_lo);
    const float near = k == 0 ? f - Rs : fk * ln2_hi - ((Rs - (fk * ln2_lo + c)) - f);
    // the general case
    const float s = f / (2.0f + f), z = s * s;
    const float R = z * (Lp1 + z * (Lp2 + z * (Lp3 + z * (Lp4 + z * (Lp5 + z * (Lp6 + z * Lp7))))));
    const float general = k == 0 ? f - (hfsq - s * (hfsq + R)) : fk * ln2_hi - ((hfsq - (s * (hfsq + R) + (fk * ln2_lo + c))) - f);
    return hu == 0 ? (f == zero ? near_zero : near) : general;
}

}  // namespace hmr
