// Element types and conversions shared by the kernels (and, for scalars, by host code).
//
// The conversions reproduce homura's Element::to_element (ref: src/dtype.rs:171-277) for every
// bit pattern, NaN payloads included, because the reference compares converted tensors bit for
// bit (ref: tests/rocm_copy.rs:12-70):
//   float source  -> exact f64 (a NaN turns quiet, payload kept at the top) -> target
//   target int    : truncate toward zero, saturate to i64 (NaN -> 0), wrap to the width
//   target f32    : round to nearest even; a NaN keeps its top 23 payload bits, quiet
//   target f16/bf16: through f32, then round to nearest even (two roundings on purpose)
//   target bool   : != 0 (NaN is true)
//   int source    -> i64 -> wrap / round to f32 or f64 / through f32 to a half / != 0
// Half conversions are done with integer arithmetic so that no denormal mode can change them.
#pragma once

#include <cstdint>
#include <type_traits>

#include "homura_rocm.h"

#if defined(__HIPCC__)
#include <hip/hip_runtime.h>
#define HMR_HD __host__ __device__ __forceinline__
#else
#define HMR_HD inline
#endif

namespace hmr {

// Storage types. Distinct wrappers so that overloads can tell them apart.
struct bool_t {
    uint8_t v;
};
struct f16_t {
    uint16_t bits;
};
struct bf16_t {
    uint16_t bits;
};

template <class To, class From>
HMR_HD To bits_as(From v) {
    static_assert(sizeof(To) == sizeof(From), "bits_as needs equal sizes");
    return __builtin_bit_cast(To, v);
}

enum class Kind { Bool, Int, Float };

template <int DT>
struct ElemOf;
template <>
struct ElemOf<HMR_BOOL> {
    using T = bool_t;
    static constexpr Kind kind = Kind::Bool;
};
template <>
struct ElemOf<HMR_U8> {
    using T = uint8_t;
    static constexpr Kind kind = Kind::Int;
};
template <>
struct ElemOf<HMR_I8> {
    using T = int8_t;
    static constexpr Kind kind = Kind::Int;
};
template <>
struct ElemOf<HMR_I16> {
    using T = int16_t;
    static constexpr Kind kind = Kind::Int;
};
template <>
struct ElemOf<HMR_I32> {
    using T = int32_t;
    static constexpr Kind kind = Kind::Int;
};
template <>
struct ElemOf<HMR_I64> {
    using T = int64_t;
    static constexpr Kind kind = Kind::Int;
};
template <>
struct ElemOf<HMR_F16> {
    using T = f16_t;
    static constexpr Kind kind = Kind::Float;
};
template <>
struct ElemOf<HMR_BF16> {
    using T = bf16_t;
    static constexpr Kind kind = Kind::Float;
};
template <>
struct ElemOf<HMR_F32> {
    using T = float;
    static constexpr Kind kind = Kind::Float;
};
template <>
struct ElemOf<HMR_F64> {
    using T = double;
    static constexpr Kind kind = Kind::Float;
};

HMR_HD int dtype_size(int dtype) {
    switch (dtype) {
        case HMR_BOOL:
        case HMR_U8:
        case HMR_I8: return 1;
        case HMR_I16:
        case HMR_F16:
        case HMR_BF16: return 2;
        case HMR_I32:
        case HMR_F32: return 4;
        default: return 8;
    }
}

// ---- halves <-> f32 ----------------------------------------------------------------------------

// bf16 -> f32 as arithmetic sees it: the pattern moved up. (A signalling NaN stays signalling;
// arithmetic quiets it and NaN payloads are not part of any arithmetic result's contract.)
HMR_HD float bf16_up(bf16_t h) { return bits_as<float>(static_cast<uint32_t>(h.bits) << 16); }

// bf16 -> f32 as a conversion: additionally quiets a NaN.
HMR_HD float bf16_widen(bf16_t h) {
    uint32_t b = h.bits;
    if ((b & 0x7FFFu) > 0x7F80u) b |= 0x0040u;
    return bits_as<float>(b << 16);
}

// f32 -> bf16, nearest even; NaN keeps the top 7 payload bits and turns quiet.
HMR_HD bf16_t bf16_round(float f) {
#if defined(__HIP_DEVICE_COMPILE__)
    // gfx950 converts in hardware (v_cvt_pk_bf16_f32) with the same bits for every f32 pattern, NaNs
    // included. Written as the instruction itself: the compiler's own lowering of a float -> __bf16
    // cast pairs neighbouring conversions into vector operations that this build (packed FP32
    // instructions off) cannot always select.
    uint32_t packed;
    asm("v_cvt_pk_bf16_f32 %0, %1, 0" : "=v"(packed) : "v"(f));
    return bf16_t{static_cast<uint16_t>(packed)};
#endif
    uint32_t x = bits_as<uint32_t>(f);
    if ((x & 0x7FFFFFFFu) > 0x7F800000u) return bf16_t{static_cast<uint16_t>((x >> 16) | 0x0040u)};
    return bf16_t{static_cast<uint16_t>((x + 0x7FFFu + ((x >> 16) & 1u)) >> 16)};
}

// Two f32 values rounded to bf16 and packed (lo in bits 0-15): one instruction on the device.
HMR_HD uint32_t bf16_round_pair(float lo, float hi) {
#if defined(__HIP_DEVICE_COMPILE__)
    uint32_t packed;
    asm("v_cvt_pk_bf16_f32 %0, %1, %2" : "=v"(packed) : "v"(lo), "v"(hi));
    return packed;
#else
    return static_cast<uint32_t>(bf16_round(lo).bits) | (static_cast<uint32_t>(bf16_round(hi).bits) << 16);
#endif
}

// f16 -> f32, exact, by integer arithmetic. NaN: quiet, payload at the top of the mantissa.
HMR_HD float f16_widen(f16_t h) {
#if defined(__HIP_DEVICE_COMPILE__)
    // v_cvt_f32_f16: same bits for all 65 536 patterns. As the instruction itself, so that the compiler
    // cannot fold the conversion into a mixed-precision multiply-add (x * s became fma(x, s, +0), which
    // turns -0 into +0).
    float f;
    asm("v_cvt_f32_f16 %0, %1" : "=v"(f) : "v"(static_cast<uint32_t>(h.bits)));
    return f;
#endif
    uint32_t sign = static_cast<uint32_t>(h.bits & 0x8000u) << 16;
    uint32_t exp = (h.bits >> 10) & 0x1Fu;
    uint32_t man = h.bits & 0x3FFu;
    uint32_t out;
    if (exp == 0x1Fu) {
        out = man == 0 ? 0x7F800000u : (0x7FC00000u | (man << 13));
    } else if (exp != 0) {
        out = ((exp + 112u) << 23) | (man << 13);
    } else if (man == 0) {
        out = 0;
    } else {
        // Subnormal man * 2^-24: shift the leading one up to bit 10.
        int lead = 31 - __builtin_clz(man);  // 0..9
        int shift = 10 - lead;
        out = (static_cast<uint32_t>(113 - shift) << 23) | (((man << shift) & 0x3FFu) << 13);
    }
    return bits_as<float>(sign | out);
}

// f32 -> f16, nearest even; NaN keeps the top 10 payload bits and turns quiet.
HMR_HD f16_t f16_round(float f) {
#if defined(__HIP_DEVICE_COMPILE__)
    uint32_t hw;  // v_cvt_f16_f32: same bits for every f32 pattern
    asm("v_cvt_f16_f32 %0, %1" : "=v"(hw) : "v"(f));
    return f16_t{static_cast<uint16_t>(hw)};
#endif
    uint32_t x = bits_as<uint32_t>(f);
    uint32_t sign = (x >> 16) & 0x8000u;
    uint32_t a = x & 0x7FFFFFFFu;
    uint32_t h;
    if (a > 0x7F800000u) {
        h = 0x7E00u | ((a >> 13) & 0x3FFu);
    } else if (a >= 0x47800000u) {  // >= 2^16, infinities included
        h = 0x7C00u;
    } else if (a >= 0x38800000u) {  // normal f16 range (>= 2^-14)
        uint32_t m = a & 0x7FFFFFu;
        h = (((a >> 23) - 112u) << 10) | (m >> 13);
        uint32_t rem = m & 0x1FFFu;
        h += (rem > 0x1000u || (rem == 0x1000u && (h & 1u))) ? 1u : 0u;
    } else if (a < 0x33000000u) {  // < 2^-25: rounds to zero (2^-25 itself is a tie to even)
        h = 0;
    } else {
        uint32_t m = (a & 0x7FFFFFu) | 0x800000u;
        uint32_t s = 126u - (a >> 23);  // 14..24: units of 2^-24 are m >> s
        h = m >> s;
        uint32_t rem = m & ((1u << s) - 1u);
        uint32_t half = 1u << (s - 1u);
        h += (rem > half || (rem == half && (h & 1u))) ? 1u : 0u;
    }
    return f16_t{static_cast<uint16_t>(sign | h)};
}

// ---- float -> i64 (Rust's `as i64`) and wrapping ------------------------------------------------

HMR_HD int64_t f64_to_i64_sat(double v) {
    if (v != v) return 0;
    if (v >= 9223372036854775808.0) return INT64_MAX;
    if (v <= -9223372036854775808.0) return INT64_MIN;
    return static_cast<int64_t>(v);
}

template <class T>
HMR_HD T wrap_to(int64_t v) {
    using U = std::make_unsigned_t<T>;
    return bits_as<T>(static_cast<U>(static_cast<uint64_t>(v)));
}

// ---- Sealed conversions per element type --------------------------------------------------------

template <class T>
struct Conv;

#define HMR_INT_CONV(T)                                                              \
    template <>                                                                      \
    struct Conv<T> {                                                                 \
        static constexpr Kind kind = Kind::Int;                                      \
        static HMR_HD double to_f64(T v) { return static_cast<double>(v); }          \
        static HMR_HD int64_t to_i64(T v) { return static_cast<int64_t>(v); }        \
        static HMR_HD bool to_bool(T v) { return v != 0; }                           \
        static HMR_HD T from_f64(double v) { return wrap_to<T>(f64_to_i64_sat(v)); } \
        static HMR_HD T from_i64(int64_t v) { return wrap_to<T>(v); }                \
        static HMR_HD T from_bool(bool v) { return static_cast<T>(v ? 1 : 0); }      \
    };
HMR_INT_CONV(uint8_t)
HMR_INT_CONV(int8_t)
HMR_INT_CONV(int16_t)
HMR_INT_CONV(int32_t)
HMR_INT_CONV(int64_t)
#undef HMR_INT_CONV

template <>
struct Conv<bool_t> {
    static constexpr Kind kind = Kind::Bool;
    static HMR_HD double to_f64(bool_t v) { return v.v ? 1.0 : 0.0; }
    static HMR_HD int64_t to_i64(bool_t v) { return v.v ? 1 : 0; }
    static HMR_HD bool to_bool(bool_t v) { return v.v != 0; }
    static HMR_HD bool_t from_f64(double v) { return bool_t{static_cast<uint8_t>(v != 0.0)}; }
    static HMR_HD bool_t from_i64(int64_t v) { return bool_t{static_cast<uint8_t>(v != 0)}; }
    static HMR_HD bool_t from_bool(bool v) { return bool_t{static_cast<uint8_t>(v)}; }
};

template <>
struct Conv<float> {
    static constexpr Kind kind = Kind::Float;
    static HMR_HD double to_f64(float v) { return static_cast<double>(v); }
    static HMR_HD int64_t to_i64(float v) { return f64_to_i64_sat(static_cast<double>(v)); }
    static HMR_HD bool to_bool(float v) { return v != 0.0f; }
    static HMR_HD float from_f64(double v) { return static_cast<float>(v); }
    static HMR_HD float from_i64(int64_t v) { return static_cast<float>(v); }
    static HMR_HD float from_bool(bool v) { return v ? 1.0f : 0.0f; }
};

template <>
struct Conv<double> {
    static constexpr Kind kind = Kind::Float;
    static HMR_HD double to_f64(double v) { return v; }
    static HMR_HD int64_t to_i64(double v) { return f64_to_i64_sat(v); }
    static HMR_HD bool to_bool(double v) { return v != 0.0; }
    static HMR_HD double from_f64(double v) { return v; }
    static HMR_HD double from_i64(int64_t v) { return static_cast<double>(v); }
    static HMR_HD double from_bool(bool v) { return v ? 1.0 : 0.0; }
};

template <>
struct Conv<f16_t> {
    static constexpr Kind kind = Kind::Float;
    static HMR_HD double to_f64(f16_t v) { return static_cast<double>(f16_widen(v)); }
    static HMR_HD int64_t to_i64(f16_t v) { return f64_to_i64_sat(static_cast<double>(f16_widen(v))); }
    static HMR_HD bool to_bool(f16_t v) { return (v.bits & 0x7FFFu) != 0; }
    static HMR_HD f16_t from_f64(double v) { return f16_round(static_cast<float>(v)); }
    static HMR_HD f16_t from_i64(int64_t v) { return f16_round(static_cast<float>(v)); }
    static HMR_HD f16_t from_bool(bool v) { return f16_t{static_cast<uint16_t>(v ? 0x3C00 : 0)}; }
};

template <>
struct Conv<bf16_t> {
    static constexpr Kind kind = Kind::Float;
    static HMR_HD double to_f64(bf16_t v) { return static_cast<double>(bf16_widen(v)); }
    static HMR_HD int64_t to_i64(bf16_t v) { return f64_to_i64_sat(static_cast<double>(bf16_widen(v))); }
    static HMR_HD bool to_bool(bf16_t v) { return (v.bits & 0x7FFFu) != 0; }
    static HMR_HD bf16_t from_f64(double v) { return bf16_round(static_cast<float>(v)); }
    static HMR_HD bf16_t from_i64(int64_t v) { return bf16_round(static_cast<float>(v)); }
    static HMR_HD bf16_t from_bool(bool v) { return bf16_t{static_cast<uint16_t>(v ? 0x3F80 : 0)}; }
};

// Element::to_element.
template <class D, class S>
HMR_HD D convert(S x) {
    if constexpr (std::is_same_v<D, S>) {
        return x;
    } else if constexpr (Conv<S>::kind == Kind::Float) {
        return Conv<D>::from_f64(Conv<S>::to_f64(x));
    } else if constexpr (Conv<S>::kind == Kind::Int) {
        return Conv<D>::from_i64(Conv<S>::to_i64(x));
    } else {
        return Conv<D>::from_bool(Conv<S>::to_bool(x));
    }
}

// ---- computation type of a float element (ref: src/backend/cpu/num.rs:53-107) ------------------

template <class T>
struct Comp;
template <>
struct Comp<float> {
    using C = float;
    static HMR_HD float up(float v) { return v; }
    static HMR_HD float down(float c) { return c; }
};
template <>
struct Comp<double> {
    using C = double;
    static HMR_HD double up(double v) { return v; }
    static HMR_HD double down(double c) { return c; }
};
template <>
struct Comp<f16_t> {
    using C = float;
    static HMR_HD float up(f16_t v) { return f16_widen(v); }
    static HMR_HD f16_t down(float c) { return f16_round(c); }
};
template <>
struct Comp<bf16_t> {
    using C = float;
    static HMR_HD float up(bf16_t v) { return bf16_up(v); }
    static HMR_HD bf16_t down(float c) { return bf16_round(c); }
};

}  // namespace hmr
