// sin, cos and log for f32 values the way the host's C library computes sinf, cosf and logf, so that the ops of
// those names get the CPU's bits (ref: src/backend/cpu/mod.rs:378-403: f32::sin, f32::cos and f32::ln, that is
// libm's). glibc's routines (2.28 and later) are those of Arm's optimized-routines (math/sinf.c, cosf.c,
// sincosf.h, logf.c and their data; MIT licence, Copyright (c) 2017-2018 Arm Limited), evaluated in f64 and
// rounded once, restated here from their published algorithms:
//   sin, cos   |x| < pi/4: odd and even polynomials in x (degree 7 and 8). Up to 120: n = round(x 2/pi) from a
//              product scaled by 2^24, x - n pi/2 in f64, the polynomial by quadrant. Beyond: the 24-bit
//              significand times 96 bits of 2/pi picked by the exponent, the top two bits of the product's
//              fraction the quadrant, the rest the reduced argument.
//   log        x = 2^k z with z in [0.7, 1.4), 16 subintervals with c near each centre: log x = k ln 2 + log c +
//              log1p(z / c - 1), a cubic in r = z / c - 1.
// The host library is built with and without fused multiply-adds and picks by its CPU; FUSED restates the first
// build, which every x86-64 core this library runs beside takes. Compared with the host's functions over all 2^32
// inputs (tests/libm_check.cpp), the fused forms differ for none (the unfused sinf for 12, cosf for 22, logf for
// none); the same comparison pins every constant. The table of 2/pi is recomputed from pi, not copied.
//
// Plain C++ apart from the fused multiply-add builtin, so a host program compiles it.
#pragma once
#include <cstdint>
#include <cstring>

namespace hmr {

template <bool FUSED>
__host__ __device__ __forceinline__ double libm_mad(double a, double b, double c) {
    if constexpr (FUSED) {
        return __builtin_fma(a, b, c);
    } else {
        volatile double p = a * b;  // a product rounded on its own, whatever the compiler would rather do
        return p + c;
    }
}

__host__ __device__ __forceinline__ uint32_t libm_top12(float x) {
    uint32_t b;
    memcpy(&b, &x, 4);
    return (b >> 20) & 0x7ff;
}

// The polynomial of quadrant n for a reduced argument x (x2 = x^2): sine for even n, cosine for odd; `negated`
// flips the cosine (the second half of the circle).
template <bool FUSED>
__host__ __device__ __forceinline__ float sincos_poly(double x, double x2, int n, bool negated) {
    constexpr double c0 = 0x1p0, c1 = -0x1.ffffffd0c621cp-2, c2 = 0x1.55553e1068f19p-5, c3 = -0x1.6c087e89a359dp-10,
                     c4 = 0x1.99343027bf8c3p-16;
    constexpr double s1 = -0x1.555545995a603p-3, s2 = 0x1.1107605230bc4p-7, s3 = -0x1.994eb3774cf24p-13;
    if ((n & 1) == 0) {
        const double x3 = x * x2, t = libm_mad<FUSED>(x2, s3, s2), x7 = x3 * x2, s = libm_mad<FUSED>(x3, s1, x);
        return static_cast<float>(libm_mad<FUSED>(x7, t, s));
    }
    const double x4 = x2 * x2, u = libm_mad<FUSED>(x2, c4, c3), v = libm_mad<FUSED>(x2, c1, c0), x6 = x4 * x2,
                 c = libm_mad<FUSED>(x4, c2, v);
    const double r = libm_mad<FUSED>(x6, u, c);  // with every coefficient negated the same roundings, negated
    return static_cast<float>(negated ? -r : r);
}

// x - n pi/2 for |x| < 120 and the quadrant n.
template <bool FUSED>
__host__ __device__ __forceinline__ double sincos_reduce(double x, int &n) {
    constexpr double kTwoOverPi24 = 0x1.45F306DC9C883p+23, kHalfPi = 0x1.921FB54442D18p0;
    const double r = x * kTwoOverPi24;
    n = (static_cast<int32_t>(r) + 0x800000) >> 24;
    return libm_mad<FUSED>(-static_cast<double>(n), kHalfPi, x);
}

// The same for 120 <= |x| < inf from the bits of x.
__host__ __device__ __forceinline__ double sincos_reduce_large(uint32_t xi, int &n) {
    // Bits of 2/pi: entry i holds the 32 bits that end 8 i bits after the binary point.
    static constexpr uint32_t kTwoOverPi[24] = {0xa2,       0xa2f9,     0xa2f983,   0xa2f9836e, 0xf9836e4e, 0x836e4e44,
                                                0x6e4e4415, 0x4e441529, 0x441529fc, 0x1529fc27, 0x29fc2757, 0xfc2757d1,
                                                0x2757d1f5, 0x57d1f534, 0xd1f534dd, 0xf534ddc0, 0x34ddc0db, 0xddc0db62,
                                                0xc0db6295, 0xdb629599, 0x6295993c, 0x95993c43, 0x993c4390, 0x3c439041};
    const uint32_t *arr = &kTwoOverPi[(xi >> 26) & 15];
    const int shift = (xi >> 23) & 7;
    xi = (xi & 0xffffff) | 0x800000;
    xi <<= shift;
    uint64_t res0 = xi * arr[0];  // 32-bit product: the bits above go into whole turns
    const uint64_t res1 = static_cast<uint64_t>(xi) * arr[4], res2 = static_cast<uint64_t>(xi) * arr[8];
    res0 = (res2 >> 32) | (res0 << 32);
    res0 += res1;
    const uint64_t q = (res0 + (uint64_t{1} << 61)) >> 62;
    res0 -= q << 62;
    n = static_cast<int>(q);
    return static_cast<double>(static_cast<int64_t>(res0)) * 0x1.921FB54442D18p-62;
}

template <bool FUSED, bool COS>
__host__ __device__ __forceinline__ float sincosf_like_libm(float y) {
    double x = y;
    int n;
    const uint32_t top = libm_top12(y);
    if (top < libm_top12(0x1.921FB6p-1f)) {  // |y| < pi/4
        if (top < libm_top12(0x1p-12f)) return COS ? 1.0f : y;
        return sincos_poly<FUSED>(x, x * x, COS ? 1 : 0, false);
    }
    bool second_half;
    if (top < libm_top12(120.0f)) {
        x = sincos_reduce<FUSED>(x, n);
        second_half = (n & 2) != 0;
        x = ((n & 3) == 1 || (n & 3) == 2) ? -x : x;  // signs +, -, -, + by quadrant
    } else if (top < 0x7f8) {
        uint32_t xi;
        memcpy(&xi, &y, 4);
        const int sign = static_cast<int>(xi >> 31);
        x = sincos_reduce_large(xi, n);
        const int q = n + sign;
        second_half = (q & 2) != 0;
        x = ((q & 3) == 1 || (q & 3) == 2) ? -x : x;
    } else {
        return (y - y) / (y - y);  // an infinity or a NaN
    }
    return sincos_poly<FUSED>(x, x * x, COS ? n ^ 1 : n, second_half);
}

template <bool FUSED>
__host__ __device__ __forceinline__ float logf_like_libm(float x) {
    // {1 / c, log c} for the sixteen subintervals of [0.7, 1.4).
    static constexpr double kTable[16][2] = {
        {0x1.661ec79f8f3bep+0, -0x1.57bf7808caadep-2}, {0x1.571ed4aaf883dp+0, -0x1.2bef0a7c06ddbp-2},
        {0x1.49539f0f010bp+0, -0x1.01eae7f513a67p-2},  {0x1.3c995b0b80385p+0, -0x1.b31d8a68224e9p-3},
        {0x1.30d190c8864a5p+0, -0x1.6574f0ac07758p-3}, {0x1.25e227b0b8eap+0, -0x1.1aa2bc79c81p-3},
        {0x1.1bb4a4a1a343fp+0, -0x1.a4e76ce8c0e5ep-4}, {0x1.12358f08ae5bap+0, -0x1.1973c5a611cccp-4},
        {0x1.0953f419900a7p+0, -0x1.252f438e10c1ep-5}, {0x1p+0, 0x0p+0},
        {0x1.e608cfd9a47acp-1, 0x1.aa5aa5df25984p-5},  {0x1.ca4b31f026aap-1, 0x1.c5e53aa362eb4p-4},
        {0x1.b2036576afce6p-1, 0x1.526e57720db08p-3},  {0x1.9c2d163a1aa2dp-1, 0x1.bc2860d22477p-3},
        {0x1.886e6037841edp-1, 0x1.1058bc8a07ee1p-2},  {0x1.767dcf5534862p-1, 0x1.4043057b6ee09p-2}};
    constexpr double kLn2 = 0x1.62e42fefa39efp-1, kA0 = -0x1.00ea348b88334p-2, kA1 = 0x1.5575b0be00b6ap-2,
                     kA2 = -0x1.ffffef20a4123p-2;
    uint32_t ix;
    memcpy(&ix, &x, 4);
    if (ix == 0x3f800000u) return 0.0f;
    if (ix - 0x00800000u >= 0x7f800000u - 0x00800000u) {  // below 2^-126, negative, infinite or a NaN
        if (ix * 2 == 0) return -__builtin_inff();
        if (ix == 0x7f800000u) return x;
        if ((ix & 0x80000000u) || ix * 2 >= 0xff000000u) return (x - x) / (x - x);
        const float scaled = x * 0x1p23f;  // a subnormal
        memcpy(&ix, &scaled, 4);
        ix -= 23u << 23;
    }
    const uint32_t tmp = ix - 0x3f330000u;
    const int i = (tmp >> 19) % 16;
    const int k = static_cast<int32_t>(tmp) >> 23;
    const uint32_t iz = ix - (tmp & 0xff800000u);
    float zf;
    memcpy(&zf, &iz, 4);
    const double z = zf;
    const double r = libm_mad<FUSED>(z, kTable[i][0], -1.0);
    const double y0 = libm_mad<FUSED>(static_cast<double>(k), kLn2, kTable[i][1]);
    const double r2 = r * r;
    double y = libm_mad<FUSED>(kA1, r, kA2);
    y = libm_mad<FUSED>(kA0, r2, y);
    y = libm_mad<FUSED>(y, r2, y0 + r);
    return static_cast<float>(y);
}

}  // namespace hmr
