// The Box-Muller pair of hmr_random_normal for outputs of at most 32 bits (ref: src/ops/random.rs:203-216, the
// CPU's `normal`: r = sqrt(-2 ln u1), theta = 2 pi u2, the cosine first): f64 polynomials in place of the
// library's log, sqrt, sin and cos. Every piece is good to about 2^-50 of its value. One output ulp would ask for
// far less, but a sample is mean + std * z, and where the two cancel the result and its ulp are small while the
// error of std * z is not: the class the samples are held to, 6 * 2^-53 times (|mean| + |std| r (1 + 2 pi)) plus
// one output ulp (ref: tests/rocm_random.rs:145-222), is an f64 evaluation's. (With pieces good to 2^-38 one f32
// sample in some millions of normal(3, 10) left it.) An f64 output keeps the library functions.
//
// The file is plain C++ apart from the two hardware estimates, which the caller brings in as `Seeds`
// (rcp and rsq, each good to 2^-22 at least), so a host program can run the same arithmetic.
#pragma once
#include <cstdint>
#include <cstring>

namespace hmr {

// ln(u) for a normal u in (0, 1]: u = 2^e m with m in [sqrt(1/2), sqrt(2)], ln m = 2 atanh(s) with
// s = (m - 1) / (m + 1), |s| <= 0.1716. The series stops after s^20 / 21; what it leaves out is
// below 1e-18 of the sum. u near 1 has e = 0, so the result keeps its relative accuracy there.
template <class Seeds>
__host__ __device__ __forceinline__ double normal_log(double u) {
    uint64_t bits;
    memcpy(&bits, &u, 8);
    int e = static_cast<int>(bits >> 52) - 1023;
    bits = (bits & 0x000FFFFFFFFFFFFFull) | 0x3FF0000000000000ull;
    double m;
    memcpy(&m, &bits, 8);
    if (m > 1.4142135623730951) {
        m *= 0.5;
        e += 1;
    }
    const double den = m + 1.0;
    double inv = Seeds::rcp(den);
    inv = __builtin_fma(__builtin_fma(-den, inv, 1.0), inv, inv);
    inv = __builtin_fma(__builtin_fma(-den, inv, 1.0), inv, inv);  // 2^-22 -> 2^-44 -> below 2^-52
    const double s = (m - 1.0) * inv, z = s * s;
    double p = 1.0 / 21.0;
    p = __builtin_fma(p, z, 1.0 / 19.0);
    p = __builtin_fma(p, z, 1.0 / 17.0);
    p = __builtin_fma(p, z, 1.0 / 15.0);
    p = __builtin_fma(p, z, 1.0 / 13.0);
    p = __builtin_fma(p, z, 1.0 / 11.0);
    p = __builtin_fma(p, z, 1.0 / 9.0);
    p = __builtin_fma(p, z, 1.0 / 7.0);
    p = __builtin_fma(p, z, 1.0 / 5.0);
    p = __builtin_fma(p, z, 1.0 / 3.0);
    const double log_m = __builtin_fma(s * z, p, s) * 2.0;
    return __builtin_fma(static_cast<double>(e), 0.6931471805599453, log_m);
}

// sqrt(x) for a finite x >= 0: x times the estimate of 1 / sqrt(x), refined twice (2^-51). Zero, which only
// u1 = 1 gives, is taken for 1e-300: its root, 1e-150, vanishes in every output narrower than f64.
template <class Seeds>
__host__ __device__ __forceinline__ double normal_sqrt(double x_in) {
    const double x = __builtin_fmax(x_in, 1e-300);
    const double y = Seeds::rsq(x), h = 0.5 * y;
    double g = x * y;
    g = __builtin_fma(__builtin_fma(-g, g, x), h, g);
    return __builtin_fma(__builtin_fma(-g, g, x), h, g);
}

// cos and sin of 2 pi t for t in [0, 1): t = k / 4 + f exactly, |f| <= 1/8, and the pair for
// phi = 2 pi f in [-pi/4, pi/4] is turned by k quarter turns. Since f is exact, values next to a zero
// crossing keep their relative accuracy. Taylor terms to phi^17 and phi^18.
__host__ __device__ __forceinline__ void normal_turn(double t, double &cosine, double &sine) {
    const int k = static_cast<int>(__builtin_fma(t, 4.0, 0.5));
    const double f = __builtin_fma(static_cast<double>(k), -0.25, t);
    const double phi = f * 6.283185307179586, z = phi * phi;
    double s = 1.0 / 355687428096000.0;
    s = __builtin_fma(s, z, -1.0 / 1307674368000.0);
    s = __builtin_fma(s, z, 1.0 / 6227020800.0);
    s = __builtin_fma(s, z, -1.0 / 39916800.0);
    s = __builtin_fma(s, z, 1.0 / 362880.0);
    s = __builtin_fma(s, z, -1.0 / 5040.0);
    s = __builtin_fma(s, z, 1.0 / 120.0);
    s = __builtin_fma(s, z, -1.0 / 6.0);
    s = __builtin_fma(phi * z, s, phi);
    double c = -1.0 / 6402373705728000.0;
    c = __builtin_fma(c, z, 1.0 / 20922789888000.0);
    c = __builtin_fma(c, z, -1.0 / 87178291200.0);
    c = __builtin_fma(c, z, 1.0 / 479001600.0);
    c = __builtin_fma(c, z, -1.0 / 3628800.0);
    c = __builtin_fma(c, z, 1.0 / 40320.0);
    c = __builtin_fma(c, z, -1.0 / 720.0);
    c = __builtin_fma(c, z, 1.0 / 24.0);
    c = __builtin_fma(c, z, -0.5);
    c = __builtin_fma(c, z, 1.0);
    const bool swap = (k & 1) != 0;
    const double a = swap ? s : c, b = swap ? c : s;
    cosine = (((k + 1) & 2) != 0) ? -a : a;  // k = 1, 2 negate the cosine
    sine = ((k & 2) != 0) ? -b : b;          // k = 2, 3 negate the sine
}

// The pair before the affine step: r cos(theta) and r sin(theta) for u1 in (0, 1], u2 in [0, 1).
template <class Seeds>
__host__ __device__ __forceinline__ void normal_polar(double u1, double u2, double &r, double &cosine, double &sine) {
    r = normal_sqrt<Seeds>(-2.0 * normal_log<Seeds>(u1));
    normal_turn(u2, cosine, sine);
}

}  // namespace hmr
