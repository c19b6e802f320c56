// The op functors of the elementwise engine. Each mirrors one arm of homura's CPU kernels
// (ref: src/backend/cpu/mod.rs:336-507, 573-577; src/backend/cpu/num.rs:109-219): float ops widen
// to the computation type (f32 for F16/BF16/F32, f64 for F64), compute, and round once; integer
// ops wrap.
//
// Transcendental accuracy. The CPU calls the host libm in the computation type. For f32 values (F16,
// BF16 and F32 tensors) exp, log, sin, cos, tanh and log1p are the host library's expf, logf, sinf,
// cosf, tanhf and log1pf restated (expf_like_libm.hpp, f32_like_libm.hpp,
// sinf_cosf_logf_like_libm.hpp: the same bits for every one of the 2^32 inputs), so every unary op
// built on them has the CPU's bits; erf is the CPU's own f64 algorithm (ref: src/backend/cpu/num.rs:
// 30-33, 189-219), always evaluated in f64 and rounded to f32 as the CPU does, because GELU's
// 1 + erf(z) cancels for z << 0. pow of f32 values is the host library's powf restated as well
// (powf_like_libm.hpp; two arguments, so pinned by sweeps and billions of random pairs rather than by
// every input). F64 tensors: tanh (and with it gelu_tanh) is the host library's f64 tanh restated
// (f64_like_libm.hpp, pinned by sampling); the other functions are the device library's.
// The surrounding arithmetic (1/(1+e), 0.5*x*(1+t), ...) is done in the computation type in the
// CPU's order, so it contributes no difference of its own.
#pragma once

#include "elem.hpp"
#include "expf_like_libm.hpp"
#include "f32_like_libm.hpp"
#include "f64_like_libm.hpp"
#include "sinf_cosf_logf_like_libm.hpp"
#include "powf_like_libm.hpp"
#include "map.hpp"

namespace hmr {

// ---- math in the evaluation type ---------------------------------------------------------------

__device__ __forceinline__ float m_sqrt(float x) { return sqrtf(x); }  // correctly rounded
__device__ __forceinline__ double m_sqrt(double x) { return sqrt(x); }
__device__ __forceinline__ float m_abs(float x) { return fabsf(x); }
__device__ __forceinline__ double m_abs(double x) { return fabs(x); }


// exp in the computation type: for f32 (F16, BF16 and F32 tensors) the host library's own expf, bit for
// bit (expf_like_libm.hpp), because sigmoid, silu and log_sigmoid divide by or take the logarithm of
// 1 + e and turn one ulp of e into up to four of their result; for f64 the device library's exp.
template <class T>
__device__ __forceinline__ typename Comp<T>::C e_exp(typename Comp<T>::C x) {
    if constexpr (std::is_same_v<typename Comp<T>::C, float>) return expf_like_libm<true>(x);
    else return exp(x);
}
// tanh and log1p likewise (f32_like_libm.hpp): gelu_tanh's 1 + tanh cancels next to its zero, and log_sigmoid is
// a difference of which the log1p is one part.
template <class T>
__device__ __forceinline__ typename Comp<T>::C e_tanh(typename Comp<T>::C x) {
    if constexpr (std::is_same_v<typename Comp<T>::C, float>) return tanhf_like_libm(x);
    else return tanh_like_libm(x);  // f64_like_libm.hpp: the host library's, pinned by 480 million sampled inputs
}
// log, sin and cos likewise (sinf_cosf_logf_like_libm.hpp).
template <class T>
__device__ __forceinline__ typename Comp<T>::C e_log(typename Comp<T>::C x) {
    if constexpr (std::is_same_v<typename Comp<T>::C, float>) return logf_like_libm<true>(x);
    else return log(x);
}
template <class T>
__device__ __forceinline__ typename Comp<T>::C e_sin(typename Comp<T>::C x) {
    if constexpr (std::is_same_v<typename Comp<T>::C, float>) return sincosf_like_libm<true, false>(x);
    else return sin(x);
}
template <class T>
__device__ __forceinline__ typename Comp<T>::C e_cos(typename Comp<T>::C x) {
    if constexpr (std::is_same_v<typename Comp<T>::C, float>) return sincosf_like_libm<true, true>(x);
    else return cos(x);
}
template <class T>
__device__ __forceinline__ typename Comp<T>::C e_log1p(typename Comp<T>::C x) {
    if constexpr (std::is_same_v<typename Comp<T>::C, float>) return log1pf_like_libm(x);
    else return log1p(x);
}

// A NaN whose quiet bit is clear. Conversions and arithmetic quiet it, so it has to be looked for in the bits.
__device__ __forceinline__ bool is_signaling(double x) {
    const uint64_t b = static_cast<uint64_t>(__double_as_longlong(x));
    return (b & 0x7ff8000000000000ull) == 0x7ff0000000000000ull && (b & 0x0007ffffffffffffull) != 0;
}

// pow in the computation type: for f32 the host library's powf restated (powf_like_libm.hpp), which also tells a
// signaling NaN from a quiet one (x ** 0 and 1 ** y are 1 for a quiet NaN and NaN for a signaling one). The CPU
// widens a 16-bit NaN to a quiet f32 NaN before powf sees it, and bf16's widening here is a shift: quiet those.
// For f64 the device library's pow, which says 1 for both kinds of NaN, behind the same check.
template <class T>
__device__ __forceinline__ typename Comp<T>::C e_pow(typename Comp<T>::C x, typename Comp<T>::C y) {
    if constexpr (std::is_same_v<typename Comp<T>::C, float>) {
        if constexpr (sizeof(T) == 2) {
            x = x != x ? __uint_as_float(__float_as_uint(x) | 0x00400000u) : x;
            y = y != y ? __uint_as_float(__float_as_uint(y) | 0x00400000u) : y;
        }
        return powf_like_libm<true>(x, y);
    } else {
        if (is_signaling(x) || is_signaling(y)) return x + y;
        return pow(x, y);
    }
}

// erf of a computation-type value: always through f64 (see the header comment).
__device__ __forceinline__ float e_erf(float x) { return static_cast<float>(erf(static_cast<double>(x))); }

// F64 tensors: the CPU's own algorithm (ref: src/backend/cpu/num.rs:189-219), a series below 1.5
// and an 80-term continued fraction up to 6. It is only good to ~3 ulp, so an accurate erf would
// sit further from it than the same steps do; the remaining difference is the device exp's.
__device__ inline double e_erf(double x) {
    if (x != x) return x;
    const double a = fabs(x);
    double r;
    if (a < 1.5) {
        const double x2 = a * a;
        double term = a, sum = a, n = 0.0;
        while (term > 1e-17 * sum) {
            n += 1.0;
            term *= 2.0 * x2 / (2.0 * n + 1.0);
            sum += term;
        }
        r = 1.1283791670955125739 * exp(-x2) * sum;
    } else if (a < 6.0) {
        double f = a;
        for (int k = 80; k >= 1; --k) f = a + (static_cast<double>(k) * 0.5) / f;
        r = 1.0 - exp(-a * a) / (sqrt(3.14159265358979323846) * f);
    } else {
        r = 1.0;
    }
    return copysign(r, x);
}

// ---- unary ------------------------------------------------------------------------------------------

template <int OP, class T>
struct UnaryFloat {
    static constexpr int N = 1;
    using Out = T;
    using In0 = T;
    using In1 = Unused;
    using In2 = Unused;
    using C = typename Comp<T>::C;
    __device__ __forceinline__ Out operator()(T v) const {
        const C x = Comp<T>::up(v);
        const C one = C(1), zero = C(0), half = C(0.5);
        C r;
        if constexpr (OP == HMR_UNARY_NEG) r = -x;
        else if constexpr (OP == HMR_UNARY_ABS) r = m_abs(x);
        else if constexpr (OP == HMR_UNARY_SIGN) r = x > zero ? one : (x < zero ? -one : zero);
        else if constexpr (OP == HMR_UNARY_RELU) r = (x != x || x > zero) ? x : zero;
        else if constexpr (OP == HMR_UNARY_EXP) r = e_exp<T>(x);
        else if constexpr (OP == HMR_UNARY_LOG) r = e_log<T>(x);
        else if constexpr (OP == HMR_UNARY_SQRT) r = m_sqrt(x);
        else if constexpr (OP == HMR_UNARY_RSQRT) r = one / m_sqrt(x);
        else if constexpr (OP == HMR_UNARY_RECIPROCAL) r = one / x;
        else if constexpr (OP == HMR_UNARY_SIN) r = e_sin<T>(x);
        else if constexpr (OP == HMR_UNARY_COS) r = e_cos<T>(x);
        else if constexpr (OP == HMR_UNARY_ERF) r = e_erf(x);
        else if constexpr (OP == HMR_UNARY_TANH) r = e_tanh<T>(x);
        else if constexpr (OP == HMR_UNARY_SIGMOID) r = one / (one + e_exp<T>(-x));
        else if constexpr (OP == HMR_UNARY_LOG_SIGMOID) {
            C mn = (x != x || x < zero) ? x : zero;
            r = mn - e_log1p<T>(e_exp<T>(-m_abs(x)));
        } else if constexpr (OP == HMR_UNARY_SILU) r = x / (one + e_exp<T>(-x));
        else if constexpr (OP == HMR_UNARY_GELU) {
            const C k = static_cast<C>(0.70710678118654752440);
            r = half * x * (one + e_erf(x * k));
        } else {
            static_assert(OP == HMR_UNARY_GELU_TANH, "unary op");
            const C k = static_cast<C>(__builtin_sqrt(2.0 / 3.14159265358979323846));  // as the CPU: f64 sqrt(2/pi), then to C
            const C c = static_cast<C>(0.044715);
            r = half * x * (one + e_tanh<T>(k * (x + c * x * x * x)));
        }
        return Comp<T>::down(r);
    }
};

template <int OP, class T>
struct UnaryInt {
    static constexpr int N = 1;
    using Out = T;
    using In0 = T;
    using In1 = Unused;
    using In2 = Unused;
    __device__ __forceinline__ T operator()(T x) const {
        using U = std::make_unsigned_t<T>;
        if constexpr (OP == HMR_UNARY_NEG) return bits_as<T>(static_cast<U>(U(0) - static_cast<U>(x)));
        else if constexpr (OP == HMR_UNARY_ABS) {
            if constexpr (std::is_unsigned_v<T>) return x;
            else return x < 0 ? bits_as<T>(static_cast<U>(U(0) - static_cast<U>(x))) : x;
        } else if constexpr (OP == HMR_UNARY_RELU) return x > T(0) ? x : T(0);
        else {
            static_assert(OP == HMR_UNARY_SIGN, "integer unary op");
            return x > T(0) ? T(1) : (x < T(0) ? static_cast<T>(-1) : T(0));
        }
    }
};

template <class T>
struct LogicalNot {
    static constexpr int N = 1;
    using Out = bool_t;
    using In0 = T;
    using In1 = Unused;
    using In2 = Unused;
    __device__ __forceinline__ bool_t operator()(T x) const {
        return bool_t{static_cast<uint8_t>(!Conv<T>::to_bool(x))};
    }
};

// Moves elements of one size unchanged (same-dtype copies, fills, Sign of a bool tensor).
template <class W>
struct Move {
    static constexpr int N = 1;
    using Out = W;
    using In0 = W;
    using In1 = Unused;
    using In2 = Unused;
    __device__ __forceinline__ W operator()(W x) const { return x; }
};

template <class D, class S>
struct Convert {
    static constexpr int N = 1;
    using Out = D;
    using In0 = S;
    using In1 = Unused;
    using In2 = Unused;
    __device__ __forceinline__ D operator()(S x) const { return convert<D, S>(x); }
};

// ---- binary -----------------------------------------------------------------------------------------

// Value a comparison looks at: halves compare as floats, bools as 0/1.
template <class T>
__device__ __forceinline__ auto cmp_value(T x) {
    if constexpr (std::is_same_v<T, f16_t>) return f16_widen(x);
    else if constexpr (std::is_same_v<T, bf16_t>) return bf16_up(x);
    else if constexpr (std::is_same_v<T, bool_t>) return x.v;
    else return x;
}

template <int OP, class T>
struct Compare {
    static constexpr int N = 2;
    using Out = bool_t;
    using In0 = T;
    using In1 = T;
    using In2 = Unused;
    __device__ __forceinline__ bool_t operator()(T a, T b) const {
        auto x = cmp_value(a);
        auto y = cmp_value(b);
        bool r;
        if constexpr (OP == HMR_BINARY_GREATER) r = x > y;
        else if constexpr (OP == HMR_BINARY_GREATER_EQUAL) r = x >= y;
        else if constexpr (OP == HMR_BINARY_LESS) r = x < y;
        else if constexpr (OP == HMR_BINARY_LESS_EQUAL) r = x <= y;
        else if constexpr (OP == HMR_BINARY_EQUAL) r = x == y;
        else r = x != y;
        return bool_t{static_cast<uint8_t>(r)};
    }
};

// AND: LogicalAnd, bool Mul/Minimum, bool BitwiseAnd. OR: LogicalOr, bool Add/Maximum.
template <bool AND>
struct BoolBinary {
    static constexpr int N = 2;
    using Out = bool_t;
    using In0 = bool_t;
    using In1 = bool_t;
    using In2 = Unused;
    __device__ __forceinline__ bool_t operator()(bool_t a, bool_t b) const {
        bool x = a.v != 0, y = b.v != 0;
        return bool_t{static_cast<uint8_t>(AND ? (x && y) : (x || y))};
    }
};

template <class T>
__device__ __forceinline__ T wrapping_mul(T a, T b) {
    using U = std::make_unsigned_t<T>;
    using W = std::conditional_t<sizeof(T) == 8, uint64_t, uint32_t>;
    return bits_as<T>(static_cast<U>(static_cast<W>(static_cast<U>(a)) * static_cast<W>(static_cast<U>(b))));
}

// ref: src/backend/cpu/num.rs:160-187
template <class T>
__device__ __forceinline__ T int_pow(T base, T exp) {
    int64_t e = static_cast<int64_t>(exp);
    if (e < 0) {
        int64_t b = static_cast<int64_t>(base);
        if (b == 1) return T(1);
        if (b == -1) return (e % 2 == 0) ? T(1) : base;
        return T(0);
    }
    T result = 1;
    uint64_t k = static_cast<uint64_t>(e);
    while (k > 0) {
        if (k & 1) result = wrapping_mul(result, base);
        base = wrapping_mul(base, base);
        k >>= 1;
    }
    return result;
}

template <int OP, class T>
struct IntBinary {
    static constexpr int N = 2;
    using Out = T;
    using In0 = T;
    using In1 = T;
    using In2 = Unused;
    __device__ __forceinline__ T operator()(T a, T b) const {
        using U = std::make_unsigned_t<T>;
        if constexpr (OP == HMR_BINARY_ADD) return bits_as<T>(static_cast<U>(static_cast<U>(a) + static_cast<U>(b)));
        else if constexpr (OP == HMR_BINARY_SUB) return bits_as<T>(static_cast<U>(static_cast<U>(a) - static_cast<U>(b)));
        else if constexpr (OP == HMR_BINARY_MUL) return wrapping_mul(a, b);
        else if constexpr (OP == HMR_BINARY_POW) return int_pow(a, b);
        else if constexpr (OP == HMR_BINARY_MAXIMUM) return a > b ? a : b;
        else if constexpr (OP == HMR_BINARY_MINIMUM) return a < b ? a : b;
        else {
            static_assert(OP == HMR_BINARY_BITWISE_AND, "integer binary op");
            return static_cast<T>(a & b);
        }
    }
};

// A and B may differ from T (mixed-dtype extension): both are converted exactly to T's
// computation type, which is what a separate cast kernel followed by the op would produce.
template <int OP, class T, class A = T, class B = T>
struct FloatBinary {
    static constexpr int N = 2;
    using Out = T;
    using In0 = A;
    using In1 = B;
    using In2 = Unused;
    using C = typename Comp<T>::C;
    __device__ __forceinline__ T operator()(A a, B b) const {
        const C x = static_cast<C>(Comp<A>::up(a));
        const C y = static_cast<C>(Comp<B>::up(b));
        C r;
        if constexpr (OP == HMR_BINARY_ADD) r = x + y;
        else if constexpr (OP == HMR_BINARY_SUB) r = x - y;
        else if constexpr (OP == HMR_BINARY_MUL) r = x * y;
        else if constexpr (OP == HMR_BINARY_DIV) r = x / y;
        else if constexpr (OP == HMR_BINARY_POW) r = e_pow<T>(x, y);
        else if constexpr (OP == HMR_BINARY_MAXIMUM) r = (x != x || x > y) ? x : y;
        else {
            static_assert(OP == HMR_BINARY_MINIMUM, "float binary op");
            r = (x != x || x < y) ? x : y;
        }
        return Comp<T>::down(r);
    }
};

// hmr_binary_scalar: the scalar stays in the computation type (it travels as a kernel constant
// holding the bits of a C value in input 1). MODE 0: a*s, 1: a/s, 2: s/a.
template <int MODE, class T>
struct ScalarBinary {
    static constexpr int N = 2;
    using Out = T;
    using In0 = T;
    using In1 = typename Comp<T>::C;
    using In2 = Unused;
    static constexpr uint32_t kConstantInputs = 2;  // input 1 is never a tensor: its width does not shape the tiles
    using C = typename Comp<T>::C;
    __device__ __forceinline__ T operator()(T a, C s) const {
        const C x = Comp<T>::up(a);
        if constexpr (MODE == 0) return Comp<T>::down(x * s);
        else if constexpr (MODE == 1) return Comp<T>::down(x / s);
        else return Comp<T>::down(s / x);
    }
};

// ---- the optimizers' fused steps (ref: src/backend/cpu/mod.rs:509-569) -------------------------------
//
// One rounding to the dtype; the multiply-adds are fused exactly where the CPU's mul_add is. The
// coefficient arrives in the computation type (the bits of a C value).
template <int OP, class T, bool SMALL>
struct FusedStep {
    static constexpr int N = OP <= HMR_FUSED_LERP ? 2 : 3;
    using Out = T;
    using In0 = T;
    using In1 = T;
    using In2 = std::conditional_t<N == 3, T, Unused>;
    using C = typename Comp<T>::C;
    C coefficient;
    __device__ __forceinline__ explicit FusedStep(uint64_t bits) { __builtin_memcpy(&coefficient, &bits, sizeof(C)); }
    static __device__ __forceinline__ C fused(C a, C b, C c) {
        if constexpr (std::is_same_v<C, float>) return __builtin_fmaf(a, b, c);
        else return __builtin_fma(a, b, c);
    }
    __device__ __forceinline__ T operator()(T a, T b) const {
        const C x = Comp<T>::up(a), y = Comp<T>::up(b);
        if constexpr (OP == HMR_FUSED_SCALED_ADD) return Comp<T>::down(fused(y, coefficient, x));
        else return Comp<T>::down(fused(coefficient, y - x, SMALL ? x : y));
    }
    __device__ __forceinline__ T operator()(T a, T b, T c) const {
        const C x = Comp<T>::up(a), y = Comp<T>::up(b), z = Comp<T>::up(c);
        if constexpr (OP == HMR_FUSED_ADDCMUL) return Comp<T>::down(fused(coefficient * y, z, x));
        else return Comp<T>::down(x + coefficient * y / z);
    }
};

// ---- addr (ref: src/backend/cpu/linalg.rs:238-360) -----------------------------------------------------
//
// out = f(v1[i], v2[j], input[i][j]) with every step rounded to the dtype; READS = false leaves the
// input out (beta is zero). alpha and beta arrive as bits of the computation type (floats) or as i64.
template <class T, bool READS>
struct AddrFloat {
    static constexpr int N = READS ? 3 : 2;
    using Out = T;
    using In0 = T;
    using In1 = T;
    using In2 = std::conditional_t<READS, T, Unused>;
    using C = typename Comp<T>::C;
    C alpha, beta;
    __device__ __forceinline__ AddrFloat(uint64_t a, uint64_t b) {
        __builtin_memcpy(&alpha, &a, sizeof(C));
        __builtin_memcpy(&beta, &b, sizeof(C));
    }
    __device__ __forceinline__ T product(T x, T y) const {
        const T a = alpha == C(1) ? x : Comp<T>::down(Comp<T>::up(x) * alpha);
        return Comp<T>::down(Comp<T>::up(a) * Comp<T>::up(y));
    }
    __device__ __forceinline__ T operator()(T x, T y) const { return product(x, y); }
    __device__ __forceinline__ T operator()(T x, T y, T c) const {
        const T p = product(x, y);
        const T scaled = beta == C(1) ? c : Comp<T>::down(Comp<T>::up(c) * beta);
        return Comp<T>::down(Comp<T>::up(scaled) + Comp<T>::up(p));
    }
};

// Wrapping arithmetic in the element's width, which has the values of the CPU's wrapping i64
// arithmetic truncated once.
template <class T, bool READS>
struct AddrInt {
    static constexpr int N = READS ? 3 : 2;
    using Out = T;
    using In0 = T;
    using In1 = T;
    using In2 = std::conditional_t<READS, T, Unused>;
    // At least 32 bits, so that no product is promoted to a signed int that could overflow.
    using U = std::conditional_t<(sizeof(T) < 4), uint32_t, std::make_unsigned_t<T>>;
    U alpha, beta;
    __device__ __forceinline__ AddrInt(uint64_t a, uint64_t b) : alpha(static_cast<U>(a)), beta(static_cast<U>(b)) {}
    __device__ __forceinline__ U product(T x, T y) const {
        return static_cast<U>(static_cast<U>(static_cast<U>(x) * static_cast<U>(y)) * alpha);
    }
    __device__ __forceinline__ T operator()(T x, T y) const { return static_cast<T>(product(x, y)); }
    __device__ __forceinline__ T operator()(T x, T y, T c) const {
        U p = product(x, y);
        // Keeps the sum of products of bytes away from the compiler's dot-product matcher, which (ROCm 7.2,
        // gfx950) turns c * beta + (x * y) * alpha of 8-bit operands into v_dot4_u32_u8 of {x, c} and
        // {alpha, beta} plus y: the value of x * alpha + c * beta + y.
        if constexpr (sizeof(T) < 4) asm volatile("" : "+v"(p));
        return static_cast<T>(static_cast<U>(static_cast<U>(static_cast<U>(c) * beta) + p));
    }
};

template <bool READS>
struct AddrBool {
    static constexpr int N = READS ? 3 : 2;
    using Out = bool_t;
    using In0 = bool_t;
    using In1 = bool_t;
    using In2 = std::conditional_t<READS, bool_t, Unused>;
    bool alpha;
    __device__ __forceinline__ AddrBool(uint64_t a, uint64_t) : alpha(a != 0) {}
    __device__ __forceinline__ bool_t operator()(bool_t x, bool_t y) const {
        return bool_t{static_cast<uint8_t>(x.v != 0 && alpha && y.v != 0)};
    }
    __device__ __forceinline__ bool_t operator()(bool_t x, bool_t y, bool_t c) const {
        return bool_t{static_cast<uint8_t>(c.v != 0 || (x.v != 0 && alpha && y.v != 0))};
    }
};

// ---- where --------------------------------------------------------------------------------------------

template <class W>
struct Select {
    static constexpr int N = 3;
    using Out = W;
    using In0 = bool_t;
    using In1 = W;
    using In2 = W;
    __device__ __forceinline__ W operator()(bool_t c, W x, W y) const { return c.v ? x : y; }
};

}  // namespace hmr
