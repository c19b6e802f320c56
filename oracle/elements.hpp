// TEST INFRASTRUCTURE -- CPU oracle, never linked into or called from the shipped library.
//
// Element types of homura tensors and the conversions between them, restated for the host CPU
// from the reference's Rust:
//   - Element::to_element and the Sealed conversions        ref: src/dtype.rs:140-277
//   - FloatElement::{up, down}                              ref: src/backend/cpu/num.rs:55-107
//   - the `half` crate (2.7.1, not vendored in the reference) f32<->f16/bf16 conversions, whose
//     published algorithm is: widen exactly (a NaN becomes quiet and keeps its payload bits);
//     narrow with round-to-nearest-even, a NaN keeps the top payload bits and becomes quiet.
//     Pinned by the bit patterns in ref: src/dtype.rs:629-665 and the cast.* golden vectors.
//
// `x as f32`, `x as f64`, integer <-> float `as` casts of Rust are the x86-64 SSE2 conversions
// the C++ casts below compile to; `as i64` from a float saturates and maps NaN to 0, which C++
// does not define, so it is written out.
#pragma once

#include <cmath>
#include <cstdint>
#include <cstring>
#include <limits>
#include <type_traits>

namespace orc {

template <class To, class From>
inline To bit_cast(From v) {
    static_assert(sizeof(To) == sizeof(From), "size");
    To t;
    std::memcpy(&t, &v, sizeof t);
    return t;
}

struct boolean {
    uint8_t v;
};
struct f16 {
    uint16_t bits;
};
struct bf16 {
    uint16_t bits;
};

// ---- half <-> f32 ------------------------------------------------------------------------------

// Exact. A NaN comes out quiet with its 10 payload bits at the top of the f32 mantissa.
inline float f16_to_f32(f16 h) {
    uint32_t sign = static_cast<uint32_t>(h.bits & 0x8000u) << 16;
    uint32_t exp = (h.bits >> 10) & 0x1Fu;
    uint32_t man = h.bits & 0x3FFu;
    if (exp == 0x1Fu) {
        if (man == 0) return bit_cast<float>(sign | 0x7F800000u);
        return bit_cast<float>(sign | 0x7FC00000u | (man << 13));
    }
    if (exp == 0) {
        if (man == 0) return bit_cast<float>(sign);
        // Subnormal: man * 2^-24. Normalise.
        int shift = 0;
        while ((man & 0x400u) == 0) {
            man <<= 1;
            ++shift;
        }
        man &= 0x3FFu;
        uint32_t e = static_cast<uint32_t>(127 - 15 - shift + 1);
        return bit_cast<float>(sign | (e << 23) | (man << 13));
    }
    return bit_cast<float>(sign | ((exp + 127 - 15) << 23) | (man << 13));
}

// Round to nearest even. A NaN keeps its top 10 mantissa bits and becomes quiet.
inline f16 f32_to_f16(float f) {
    uint32_t x = bit_cast<uint32_t>(f);
    uint16_t sign = static_cast<uint16_t>((x >> 16) & 0x8000u);
    uint32_t a = x & 0x7FFFFFFFu;
    if (a > 0x7F800000u) return f16{static_cast<uint16_t>(sign | 0x7E00u | ((a >> 13) & 0x3FFu))};
    if (a == 0x7F800000u) return f16{static_cast<uint16_t>(sign | 0x7C00u)};
    int e = static_cast<int>(a >> 23) - 127;
    uint32_t m = a & 0x7FFFFFu;
    if (e >= 16) return f16{static_cast<uint16_t>(sign | 0x7C00u)};
    if (e >= -14) {
        uint32_t h = (static_cast<uint32_t>(e + 15) << 10) | (m >> 13);
        uint32_t rem = m & 0x1FFFu;
        if (rem > 0x1000u || (rem == 0x1000u && (h & 1u))) ++h;  // may carry up to infinity
        return f16{static_cast<uint16_t>(sign | h)};
    }
    // Below the normal range of f16: the result counts units of 2^-24.
    if ((a >> 23) == 0) return f16{sign};  // f32 zero or subnormal: far below 2^-25
    m |= 0x800000u;
    int s = -(e + 1);  // value = m * 2^(e-23) = (m >> s) units, s >= 14
    if (s > 24) return f16{sign};
    uint32_t h = m >> s;
    uint32_t rem = m & ((1u << s) - 1u);
    uint32_t half = 1u << (s - 1);
    if (rem > half || (rem == half && (h & 1u))) ++h;
    return f16{static_cast<uint16_t>(sign | h)};
}

// Exact. A NaN becomes quiet.
inline float bf16_to_f32(bf16 h) {
    uint32_t b = h.bits;
    if ((b & 0x7FFFu) > 0x7F80u) b |= 0x0040u;
    return bit_cast<float>(b << 16);
}

// Round to nearest even. A NaN keeps its top 7 mantissa bits and becomes quiet.
inline bf16 f32_to_bf16(float f) {
    uint32_t x = bit_cast<uint32_t>(f);
    if ((x & 0x7FFFFFFFu) > 0x7F800000u) return bf16{static_cast<uint16_t>((x >> 16) | 0x0040u)};
    uint32_t lsb = (x >> 16) & 1u;
    return bf16{static_cast<uint16_t>((x + 0x7FFFu + lsb) >> 16)};
}

// Rust's `v as i64` for a float: toward zero, saturating, NaN -> 0.
inline int64_t f64_as_i64(double v) {
    if (v != v) return 0;
    if (v >= 9223372036854775808.0) return std::numeric_limits<int64_t>::max();
    if (v <= -9223372036854775808.0) return std::numeric_limits<int64_t>::min();
    return static_cast<int64_t>(v);
}
inline int64_t f32_as_i64(float v) { return f64_as_i64(static_cast<double>(v)); }

// ---- the Sealed conversions of each element type (ref: src/dtype.rs:195-277) ------------------

enum class Kind { Bool, Int, Float };

template <class T>
struct El;

#define ORC_INT_ELEMENT(T, CODE)                                                         \
    template <>                                                                          \
    struct El<T> {                                                                       \
        static constexpr int code = CODE;                                                \
        static constexpr Kind kind = Kind::Int;                                          \
        static double to_f64(T v) { return static_cast<double>(v); }                     \
        static int64_t to_i64(T v) { return static_cast<int64_t>(v); }                   \
        static bool to_bool(T v) { return v != 0; }                                      \
        static T from_f64(double v) { return from_i64(f64_as_i64(v)); }                  \
        static T from_i64(int64_t v) {                                                   \
            std::make_unsigned_t<T> u = static_cast<std::make_unsigned_t<T>>(static_cast<uint64_t>(v)); \
            return bit_cast<T>(u);                                                       \
        }                                                                                \
        static T from_bool(bool v) { return static_cast<T>(v ? 1 : 0); }                 \
    };
ORC_INT_ELEMENT(uint8_t, 1)
ORC_INT_ELEMENT(int8_t, 2)
ORC_INT_ELEMENT(int16_t, 3)
ORC_INT_ELEMENT(int32_t, 4)
ORC_INT_ELEMENT(int64_t, 5)
#undef ORC_INT_ELEMENT

template <>
struct El<boolean> {
    static constexpr int code = 0;
    static constexpr Kind kind = Kind::Bool;
    static double to_f64(boolean v) { return v.v ? 1.0 : 0.0; }
    static int64_t to_i64(boolean v) { return v.v ? 1 : 0; }
    static bool to_bool(boolean v) { return v.v != 0; }
    static boolean from_f64(double v) { return boolean{static_cast<uint8_t>(v != 0.0)}; }
    static boolean from_i64(int64_t v) { return boolean{static_cast<uint8_t>(v != 0)}; }
    static boolean from_bool(bool v) { return boolean{static_cast<uint8_t>(v)}; }
};

template <>
struct El<float> {
    static constexpr int code = 8;
    static constexpr Kind kind = Kind::Float;
    static double to_f64(float v) { return static_cast<double>(v); }
    static int64_t to_i64(float v) { return f32_as_i64(v); }
    static bool to_bool(float v) { return v != 0.0f; }
    static float from_f64(double v) { return static_cast<float>(v); }
    static float from_i64(int64_t v) { return static_cast<float>(v); }
    static float from_bool(bool v) { return v ? 1.0f : 0.0f; }
};

template <>
struct El<double> {
    static constexpr int code = 9;
    static constexpr Kind kind = Kind::Float;
    static double to_f64(double v) { return v; }
    static int64_t to_i64(double v) { return f64_as_i64(v); }
    static bool to_bool(double v) { return v != 0.0; }
    static double from_f64(double v) { return v; }
    static double from_i64(int64_t v) { return static_cast<double>(v); }
    static double from_bool(bool v) { return v ? 1.0 : 0.0; }
};

// Halves convert through f32 in both directions (two roundings from f64 or an integer).
template <>
struct El<f16> {
    static constexpr int code = 6;
    static constexpr Kind kind = Kind::Float;
    static double to_f64(f16 v) { return static_cast<double>(f16_to_f32(v)); }
    static int64_t to_i64(f16 v) { return f32_as_i64(f16_to_f32(v)); }
    static bool to_bool(f16 v) { return f16_to_f32(v) != 0.0f; }
    static f16 from_f64(double v) { return f32_to_f16(static_cast<float>(v)); }
    static f16 from_i64(int64_t v) { return f32_to_f16(static_cast<float>(v)); }
    static f16 from_bool(bool v) { return f16{static_cast<uint16_t>(v ? 0x3C00 : 0)}; }
};

template <>
struct El<bf16> {
    static constexpr int code = 7;
    static constexpr Kind kind = Kind::Float;
    static double to_f64(bf16 v) { return static_cast<double>(bf16_to_f32(v)); }
    static int64_t to_i64(bf16 v) { return f32_as_i64(bf16_to_f32(v)); }
    static bool to_bool(bf16 v) { return bf16_to_f32(v) != 0.0f; }
    static bf16 from_f64(double v) { return f32_to_bf16(static_cast<float>(v)); }
    static bf16 from_i64(int64_t v) { return f32_to_bf16(static_cast<float>(v)); }
    static bf16 from_bool(bool v) { return bf16{static_cast<uint16_t>(v ? 0x3F80 : 0)}; }
};

// Element::to_element: the source's kind picks the route (ref: src/dtype.rs:186-192).
template <class D, class S>
inline D to_element(S x) {
    if constexpr (El<S>::kind == Kind::Float) {
        return El<D>::from_f64(El<S>::to_f64(x));
    } else if constexpr (El<S>::kind == Kind::Int) {
        return El<D>::from_i64(El<S>::to_i64(x));
    } else {
        return El<D>::from_bool(El<S>::to_bool(x));
    }
}

// ---- FloatElement: the computation type and the moves to and from it ---------------------------

template <class T>
struct Fl;
template <>
struct Fl<float> {
    using C = float;
    static float up(float v) { return v; }
    static float down(float c) { return c; }
};
template <>
struct Fl<double> {
    using C = double;
    static double up(double v) { return v; }
    static double down(double c) { return c; }
};
template <>
struct Fl<f16> {
    using C = float;
    static float up(f16 v) { return f16_to_f32(v); }
    static f16 down(float c) { return f32_to_f16(c); }
};
template <>
struct Fl<bf16> {
    using C = float;
    static float up(bf16 v) { return bf16_to_f32(v); }
    static bf16 down(float c) { return f32_to_bf16(c); }
};

// Comparisons of the element types as Rust's PartialOrd/PartialEq see them: halves compare by
// value (any NaN is unordered, +0 == -0), bools as false < true.
template <class T>
inline bool lt(T a, T b) {
    if constexpr (std::is_same_v<T, f16>) return f16_to_f32(a) < f16_to_f32(b);
    else if constexpr (std::is_same_v<T, bf16>) return bf16_to_f32(a) < bf16_to_f32(b);
    else if constexpr (std::is_same_v<T, boolean>) return a.v < b.v;
    else return a < b;
}
template <class T>
inline bool eq(T a, T b) {
    if constexpr (std::is_same_v<T, f16>) return f16_to_f32(a) == f16_to_f32(b);
    else if constexpr (std::is_same_v<T, bf16>) return bf16_to_f32(a) == bf16_to_f32(b);
    else if constexpr (std::is_same_v<T, boolean>) return a.v == b.v;
    else return a == b;
}
template <class T>
inline bool le(T a, T b) {
    if constexpr (std::is_same_v<T, f16>) return f16_to_f32(a) <= f16_to_f32(b);
    else if constexpr (std::is_same_v<T, bf16>) return bf16_to_f32(a) <= bf16_to_f32(b);
    else if constexpr (std::is_same_v<T, boolean>) return a.v <= b.v;
    else return a <= b;
}

}  // namespace orc
