// exp for f32 values the way the host's C library computes expf, so that the f32 operations built on it
// (exp itself, sigmoid, silu, log_sigmoid; ref: src/backend/cpu/mod.rs:378-403, which calls f32::exp, that
// is libm's expf) get the CPU's bits and not merely a correctly rounded exponential: 1 / (1 + e) turns one
// ulp of e into as much as four of the result. glibc's expf (2.27 and later) is the double-precision scheme
// of Szabolcs Nagy's optimized routines, restated here from its published description:
//   z = x * 32 / ln 2, k = round(z), r = z - k            (|r| <= 1/2)
//   exp(x) = 2^(k/32) * 2^(r/32) ~ s * (C0 r^3 + C1 r^2 + C2 r + 1),   s = 2^(k/32) from a 32-entry table
// evaluated in f64 and rounded once to f32. Its result is within 0.502 ulp of exp(x): not always the
// correctly rounded one, which is why this is a restatement and not a call of an accurate exp. The host
// library is built twice, with and without fused multiply-adds, and picks by the CPU it runs on (every
// x86-64 core this library runs beside has FMA); FUSED restates the first build. Compared with the host's
// expf over all 2^32 inputs (tests/libm_check.cpp) the fused form differs for none, the other for two; the
// same comparison pins every constant and the table.
//
// The scheme, its table and its coefficients are those of Arm's optimized-routines (math/expf.c, math/exp2f_data.c;
// MIT licence, Copyright (c) 2017-2018 Arm Limited), from which glibc took its expf; the table is recomputed here
// (2^(i/32) correctly rounded, by integer arithmetic) rather than copied.
//
// Plain C++ apart from the fused multiply-add builtin, so a host program compiles it.
#pragma once
#include <cstdint>
#include <cstring>

namespace hmr {

template <bool FUSED>
__host__ __device__ __forceinline__ double expf_mad(double a, double b, double c) {
    if constexpr (FUSED) {
        return __builtin_fma(a, b, c);
    } else {
        volatile double p = a * b;  // a product rounded on its own, whatever the compiler would rather do
        return p + c;
    }
}

// FUSED: the polynomial's multiply-adds are single roundings, as in the host library's build for CPUs with FMA.
// bits(2^(i/32)) - (i << 47) for i in 0..31: adding k << 47 to entry k % 32 yields the bits of 2^(k/32).
__host__ __device__ __forceinline__ uint64_t libm_exp2_entry(uint64_t i) {
    static constexpr uint64_t table[32] = {
        0x3ff0000000000000ull, 0x3fefd9b0d3158574ull, 0x3fefb5586cf9890full, 0x3fef9301d0125b51ull,
        0x3fef72b83c7d517bull, 0x3fef54873168b9aaull, 0x3fef387a6e756238ull, 0x3fef1e9df51fdee1ull,
        0x3fef06fe0a31b715ull, 0x3feef1a7373aa9cbull, 0x3feedea64c123422ull, 0x3feece086061892dull,
        0x3feebfdad5362a27ull, 0x3feeb42b569d4f82ull, 0x3feeab07dd485429ull, 0x3feea47eb03a5585ull,
        0x3feea09e667f3bcdull, 0x3fee9f75e8ec5f74ull, 0x3feea11473eb0187ull, 0x3feea589994cce13ull,
        0x3feeace5422aa0dbull, 0x3feeb737b0cdc5e5ull, 0x3feec49182a3f090ull, 0x3feed503b23e255dull,
        0x3feee89f995ad3adull, 0x3feeff76f2fb5e47ull, 0x3fef199bdd85529cull, 0x3fef3720dcef9069ull,
        0x3fef5818dcfba487ull, 0x3fef7c97337b9b5full, 0x3fefa4afa2a490daull, 0x3fefd0765b6e4540ull};
    return table[i];
}

template <bool FUSED>
__host__ __device__ __forceinline__ float expf_like_libm(float x) {
    uint32_t bits;
    memcpy(&bits, &x, 4);
    const uint32_t top = (bits >> 20) & 0x7ff;  // exponent and the top three fraction bits of |x|
    if (top >= 0x42b) {                         // |x| >= 88 or x is not finite
        if (bits == 0xff800000u) return 0.0f;
        if (top >= 0x7f8) return x + x;
        if (x > 0x1.62e42ep6f) return __builtin_inff();  // above ln 2^128
        if (x < -0x1.9fe368p6f) return 0.0f;             // below ln 2^-150
    }
    constexpr double kInvLn2N = 0x1.71547652b82fep+0 * 32.0;
    constexpr double kShift = 0x1.8p+52;
    constexpr double kC0 = 0x1.c6af84b912394p-5 / 32.0 / 32.0 / 32.0;
    constexpr double kC1 = 0x1.ebfce50fac4f3p-3 / 32.0 / 32.0;
    constexpr double kC2 = 0x1.62e42ff0c52d6p-1 / 32.0;
    const double z = kInvLn2N * static_cast<double>(x);
    double kd = z + kShift;  // the low bits of kd are round(z)
    uint64_t ki;
    memcpy(&ki, &kd, 8);
    kd -= kShift;
    // With FMA the product in z is not rounded before kd is taken off it: the one place where the two builds of
    // the host library differ in their results (for 2 of the 2^32 inputs).
    const double r = FUSED ? __builtin_fma(kInvLn2N, static_cast<double>(x), -kd) : z - kd;
    const uint64_t t = libm_exp2_entry(ki % 32) + (ki << 47);
    double s;
    memcpy(&s, &t, 8);
    const double p = expf_mad<FUSED>(kC0, r, kC1);
    const double r2 = r * r;
    double y = expf_mad<FUSED>(kC2, r, 1.0);
    y = expf_mad<FUSED>(p, r2, y);
    return static_cast<float>(y * s);
}

}  // namespace hmr
