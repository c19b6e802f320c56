// pow for f32 values the way the host's C library computes powf, so that pow gets the CPU's bits (ref:
// src/backend/cpu/mod.rs:573-577: f32::powf, that is libm's). glibc's powf (2.28 and later) is the one of Arm's
// optimized-routines (math/powf.c, powf_log2_data.c; MIT licence, Copyright (c) 2017-2018 Arm Limited), restated
// here from its published algorithm: log2 x from a 16-entry table and a quartic, in f64 and scaled by 32; times y;
// 2^(that / 32) from the 32-entry table that expf uses and a cubic; one rounding to f32. Zeros, infinities, NaNs
// (a signaling one gives a NaN even where a quiet one gives 1), negative bases with integer exponents and
// subnormal bases are told apart on the bits first.
//
// Two arguments: no walk over all inputs can pin this one. Compiled for the host and compared with the library's
// powf (tests/libm_check.cpp), the fused form differs for none of 26 exponents (0.5, 2, 3, -1, 1/3, 0.1, 2.5, ...,
// zeros, infinities, NaN, 1e-30, 1e30) times every 7th of the 2^32 bases and for none of 2 000 000 000 random
// pairs (half of them with exponents that are multiples of 1/64); the unfused form differs for 4 of those.
//
// Plain C++ apart from the fused multiply-add builtin, so a host program compiles it.
#pragma once
#include <cstdint>
#include <cstring>

#include "expf_like_libm.hpp"
#include "sinf_cosf_logf_like_libm.hpp"

namespace hmr {

// 0: y is no integer, 1: an odd one, 2: an even one.
__host__ __device__ __forceinline__ int powf_checkint(uint32_t iy) {
    const int e = iy >> 23 & 0xff;
    if (e < 0x7f) return 0;
    if (e > 0x7f + 23) return 2;
    if (iy & ((1u << (0x7f + 23 - e)) - 1)) return 0;
    if (iy & (1u << (0x7f + 23 - e))) return 1;
    return 2;
}
__host__ __device__ __forceinline__ bool powf_zeroinfnan(uint32_t ix) { return 2 * ix - 1 >= 2u * 0x7f800000u - 1; }
__host__ __device__ __forceinline__ bool powf_signaling(uint32_t ix) {
    return (ix & 0x7fc00000u) == 0x7f800000u && (ix & 0x003fffffu) != 0;
}

// 32 log2 of the positive normal number with the bits ix.
template <bool FUSED>
__host__ __device__ __forceinline__ double powf_log2(uint32_t ix) {
    // {1 / c, 32 log2 c} for the sixteen subintervals of [0.7, 1.4) (the same c as logf's).
    static constexpr double kTable[16][2] = {
        {0x1.661ec79f8f3bep+0, -0x1.efec65b963019p-2 * 32}, {0x1.571ed4aaf883dp+0, -0x1.b0b6832d4fca4p-2 * 32},
        {0x1.49539f0f010bp+0, -0x1.7418b0a1fb77bp-2 * 32},  {0x1.3c995b0b80385p+0, -0x1.39de91a6dcf7bp-2 * 32},
        {0x1.30d190c8864a5p+0, -0x1.01d9bf3f2b631p-2 * 32}, {0x1.25e227b0b8eap+0, -0x1.97c1d1b3b7afp-3 * 32},
        {0x1.1bb4a4a1a343fp+0, -0x1.2f9e393af3c9fp-3 * 32}, {0x1.12358f08ae5bap+0, -0x1.960cbbf788d5cp-4 * 32},
        {0x1.0953f419900a7p+0, -0x1.a6f9db6475fcep-5 * 32}, {0x1p+0, 0x0p+0 * 32},
        {0x1.e608cfd9a47acp-1, 0x1.338ca9f24f53dp-4 * 32},  {0x1.ca4b31f026aap-1, 0x1.476a9543891bap-3 * 32},
        {0x1.b2036576afce6p-1, 0x1.e840b4ac4e4d2p-3 * 32},  {0x1.9c2d163a1aa2dp-1, 0x1.40645f0c6651cp-2 * 32},
        {0x1.886e6037841edp-1, 0x1.88e9c2c1b9ff8p-2 * 32},  {0x1.767dcf5534862p-1, 0x1.ce0a44eb17bccp-2 * 32}};
    constexpr double kA0 = 0x1.27616c9496e0bp-2 * 32, kA1 = -0x1.71969a075c67ap-2 * 32, kA2 = 0x1.ec70a6ca7baddp-2 * 32,
                     kA3 = -0x1.7154748bef6c8p-1 * 32, kA4 = 0x1.71547652ab82bp0 * 32;
    const uint32_t tmp = ix - 0x3f330000u;
    const int i = (tmp >> 19) % 16;
    const uint32_t top = tmp & 0xff800000u, iz = ix - top;
    const int k = static_cast<int32_t>(top) >> (23 - 5);  // 32 times the exponent
    float zf;
    memcpy(&zf, &iz, 4);
    const double z = zf;
    const double r = libm_mad<FUSED>(z, kTable[i][0], -1.0), y0 = kTable[i][1] + static_cast<double>(k);
    const double r2 = r * r, y = libm_mad<FUSED>(kA0, r, kA1), p = libm_mad<FUSED>(kA2, r, kA3), r4 = r2 * r2;
    double q = libm_mad<FUSED>(kA4, r, y0);
    q = libm_mad<FUSED>(p, r2, q);
    return libm_mad<FUSED>(y, r4, q);
}

// 2^(xd / 32), negated when sign_bias is set (1 << 16: it lands on the sign bit).
template <bool FUSED>
__host__ __device__ __forceinline__ float powf_exp2(double xd, uint32_t sign_bias) {
    constexpr double kShift = 0x1.8p+52;
    constexpr double kC0 = 0x1.c6af84b912394p-5 / 32.0 / 32.0 / 32.0, kC1 = 0x1.ebfce50fac4f3p-3 / 32.0 / 32.0,
                     kC2 = 0x1.62e42ff0c52d6p-1 / 32.0;
    double kd = xd + kShift;
    uint64_t ki;
    memcpy(&ki, &kd, 8);
    kd -= kShift;
    const double r = xd - kd;
    const uint64_t t = libm_exp2_entry(ki % 32) + ((ki + sign_bias) << 47);
    double s;
    memcpy(&s, &t, 8);
    const double z = libm_mad<FUSED>(kC0, r, kC1), r2 = r * r;
    double y = libm_mad<FUSED>(kC2, r, 1.0);
    y = libm_mad<FUSED>(z, r2, y);
    return static_cast<float>(y * s);
}

template <bool FUSED>
__host__ __device__ __forceinline__ float powf_like_libm(float x, float y) {
    uint32_t sign_bias = 0, ix, iy;
    memcpy(&ix, &x, 4);
    memcpy(&iy, &y, 4);
    if (ix - 0x00800000u >= 0x7f800000u - 0x00800000u || powf_zeroinfnan(iy)) {
        // x below 2^-126, negative, infinite or a NaN; or y zero, infinite or a NaN.
        if (powf_zeroinfnan(iy)) {
            if (2 * iy == 0) return powf_signaling(ix) ? x + y : 1.0f;
            if (ix == 0x3f800000u) return powf_signaling(iy) ? x + y : 1.0f;
            if (2 * ix > 2u * 0x7f800000u || 2 * iy > 2u * 0x7f800000u) return x + y;
            if (2 * ix == 2 * 0x3f800000u) return 1.0f;
            if ((2 * ix < 2 * 0x3f800000u) == !(iy & 0x80000000u)) return 0.0f;  // |x| < 1 to +inf, |x| > 1 to -inf
            return y * y;
        }
        if (powf_zeroinfnan(ix)) {
            float x2 = x * x;
            if ((ix & 0x80000000u) && powf_checkint(iy) == 1) x2 = -x2;
            return (iy & 0x80000000u) ? 1 / x2 : x2;
        }
        if (ix & 0x80000000u) {  // a finite negative base
            const int yint = powf_checkint(iy);
            if (yint == 0) return (x - x) / (x - x);
            if (yint == 1) sign_bias = 1u << 16;
            ix &= 0x7fffffffu;
        }
        if (ix < 0x00800000u) {  // a subnormal base
            const float scaled = x * 0x1p23f;
            memcpy(&ix, &scaled, 4);
            ix &= 0x7fffffffu;
            ix -= 23u << 23;
        }
    }
    const double ylogx = static_cast<double>(y) * powf_log2<FUSED>(ix);
    uint64_t bits, limit;
    memcpy(&bits, &ylogx, 8);
    const double at_126 = 126.0 * 32;
    memcpy(&limit, &at_126, 8);
    if ((bits >> 47 & 0xffff) >= limit >> 47) {  // |y log2 x| >= 126
        if (ylogx > 0x1.fffffffd1d571p+6 * 32) return sign_bias ? -__builtin_inff() : __builtin_inff();
        if (ylogx <= -150.0 * 32) return sign_bias ? -0.0f : 0.0f;
    }
    return powf_exp2<FUSED>(ylogx, sign_bias);
}

}  // namespace hmr
