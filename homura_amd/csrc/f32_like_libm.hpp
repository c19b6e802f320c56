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

__host__ __device__ inline float expm1f_like_libm(float x) {
    const float one = 1.0f, tiny = 1.0e-30f, huge = 1.0e+30f;
    const float o_threshold = 8.8721679688e+01f, ln2_hi = 6.9313812256e-01f, ln2_lo = 9.0580006145e-06f, invln2 = 1.4426950216e+00f;
    const float Q1 = -3.3333335072e-02f, Q2 = 1.5873016091e-03f, Q3 = -7.9365076090e-05f, Q4 = 4.0082177293e-06f, Q5 = -2.0109921195e-07f;
    float y, hi, lo, c = 0.0f, t, e, hxs, hfx, r1;
    int32_t k;
    uint32_t hx = libm_bits(x);
    const uint32_t xsb = hx & 0x80000000u;
    hx &= 0x7fffffffu;
    if (hx >= 0x4195b844u) {
        if (hx >= 0x42b17218u) {
            if (hx > 0x7f800000u) return x + x;
            if (hx == 0x7f800000u) return xsb == 0 ? x : -1.0f;
            if (x > o_threshold) return huge * huge;
        }
        if (xsb != 0) return tiny - one;
    }
    if (hx > 0x3eb17218u) {
        if (hx < 0x3F851592u) {
            if (xsb == 0) { hi = x - ln2_hi; lo = ln2_lo; k = 1; }
            else { hi = x + ln2_hi; lo = -ln2_lo; k = -1; }
        } else {
            k = static_cast<int32_t>(invln2 * x + (xsb == 0 ? 0.5f : -0.5f));
            t = static_cast<float>(k);
            hi = x - t * ln2_hi;
            lo = t * ln2_lo;
        }
        x = hi - lo;
        c = (hi - x) - lo;
    } else if (hx < 0x33000000u) {
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
        y = libm_float(libm_bits(y) + (static_cast<uint32_t>(k) << 23));
        return y - one;
    }
    if (k < 23) {
        t = libm_float(0x3f800000u - (0x1000000u >> k));
        y = t - (e - x);
        y = libm_float(libm_bits(y) + (static_cast<uint32_t>(k) << 23));
    } else {
        t = libm_float(static_cast<uint32_t>(0x7f - k) << 23);
        y = x - (e + t);
        y += one;
        y = libm_float(libm_bits(y) + (static_cast<uint32_t>(k) << 23));
    }
    return y;
}

__host__ __device__ inline float tanhf_like_libm(float x) {
    const float one = 1.0f, two = 2.0f, tiny = 1.0e-30f;
    float t, z;
    const uint32_t jx = libm_bits(x), ix = jx & 0x7fffffffu;
    const bool neg = (jx >> 31) != 0;
    if (ix >= 0x7f800000u) return neg ? one / x - one : one / x + one;
    if (ix < 0x41b00000u) {
        if (ix == 0) return x;
        if (ix < 0x24000000u) return x * (one + x);
        const float ax = libm_float(ix);
        if (ix >= 0x3f800000u) { t = expm1f_like_libm(two * ax); z = one - two / (t + two); }
        else { t = expm1f_like_libm(-two * ax); z = -t / (t + two); }
    } else {
        z = one - tiny;
    }
    return neg ? -z : z;
}

__host__ __device__ inline float log1pf_like_libm(float x) {
    const float ln2_hi = 6.9313812256e-01f, ln2_lo = 9.0580006145e-06f, two25 = 3.355443200e+07f, zero = 0.0f;
    const float Lp1 = 6.6666668653e-01f, Lp2 = 4.0000000596e-01f, Lp3 = 2.8571429849e-01f, Lp4 = 2.2222198546e-01f,
                Lp5 = 1.8183572590e-01f, Lp6 = 1.5313838422e-01f, Lp7 = 1.4798198640e-01f;
    float hfsq, f = 0.0f, c = 0.0f, s, z, R, u;
    int32_t k, hx, hu = 0, ax;
    hx = static_cast<int32_t>(libm_bits(x));
    ax = hx & 0x7fffffff;
    k = 1;
    if (hx < 0x3ed413d7) {
        if (ax >= 0x3f800000) {
            if (x == -1.0f) return -two25 / zero;
            return (x - x) / (x - x);
        }
        if (ax < 0x31000000) {
            if (ax < 0x24800000) return x;
            return x - x * x * 0.5f;
        }
        if (hx > 0 || hx <= static_cast<int32_t>(0xbe95f61fu)) { k = 0; f = x; hu = 1; }
    }
    if (hx >= 0x7f800000) return x + x;
    if (k != 0) {
        if (hx < 0x5a000000) {
            u = 1.0f + x;
            hu = static_cast<int32_t>(libm_bits(u));
            k = (hu >> 23) - 127;
            c = (k > 0) ? 1.0f - (u - x) : x - (u - 1.0f);
            c /= u;
        } else {
            u = x;
            hu = static_cast<int32_t>(libm_bits(u));
            k = (hu >> 23) - 127;
            c = 0;
        }
        hu &= 0x007fffff;
        if (hu < 0x3504f7) {
            u = libm_float(static_cast<uint32_t>(hu) | 0x3f800000u);
        } else {
            k += 1;
            u = libm_float(static_cast<uint32_t>(hu) | 0x3f000000u);
            hu = (0x00800000 - hu) >> 2;
        }
        f = u - 1.0f;
    }
    hfsq = 0.5f * f * f;
    if (hu == 0) {
        if (f == zero) {
            if (k == 0) return zero;
            c += k * ln2_lo;
            return k * ln2_hi + c;
        }
        R = hfsq * (1.0f - 0.66666666666666666f * f);
        if (k == 0) return f - R;
        return k * ln2_hi - ((R - (k * ln2_lo + c)) - f);
    }
    s = f / (2.0f + f);
    z = s * s;
    R = z * (Lp1 + z * (Lp2 + z * (Lp3 + z * (Lp4 + z * (Lp5 + z * (Lp6 + z * Lp7))))));
    if (k == 0) return f - (hfsq - s * (hfsq + R));
    return k * ln2_hi - ((hfsq - (s * (hfsq + R) + (k * ln2_lo + c))) - f);
}

}  // namespace hmr
