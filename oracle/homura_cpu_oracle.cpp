// TEST INFRASTRUCTURE -- the CPU oracle for homura's elementwise / broadcast / reduction path.
//
// A restatement, for the host CPU, of the kernels of homura's CPU reference backend, which is
// the numerical definition the GPU kernels are held to. It is single-threaded like the
// reference (one global execution lock, ref: src/backend/cpu/mod.rs:40-64). Only tests,
// __graft_entry__.smoke() and bench.py's cpu_baseline leg may load it; the shipped library has
// no path into it.
//
// What each part follows:
//   loop-nest planning (Plan)            ref: src/backend/cpu/iter.rs:9-94
//   map0..map3, copy, fill               ref: src/backend/cpu/mod.rs:184-261, 315-332
//   unary, binary, *_constant, *_scalar  ref: src/backend/cpu/mod.rs:336-507
//   where_, where_constant               ref: src/backend/cpu/mod.rs:573-600
//   int_pow, erf                         ref: src/backend/cpu/num.rs:160-219
//   fold, reduce, var, arg_reduce        ref: src/backend/cpu/reduce.rs:10-225
//   softmax                              ref: src/backend/cpu/misc.rs:13-51
//   fused optimizer steps                ref: src/backend/cpu/mod.rs:509-569
//   addr                                 ref: src/backend/cpu/linalg.rs:224-388
//   triangle, flip                       ref: src/backend/cpu/misc.rs:347-411
//   exclusive_cumprod                    ref: src/backend/cpu/reduce.rs:286-324
//   Philox blocks, uniform, normal, int  ref: src/ops/random.rs:29-226
//   positions, index_select, gather,     ref: src/backend/cpu/misc.rs:53-127, 213-345
//   index_add, scatter_add (add_at)
//   index_overwrite, mask_coordinates,   ref: src/backend/cpu/misc.rs:104-203
//   index_positions
//   element conversions                  elements.hpp
//
// What pins each part (golden vectors of the reference, known answers, independent arithmetic) is listed
// beside the tests that do it: tests/test_golden_ops.py, test_optim_golden.py, test_gradient_golden.py,
// test_oracle_kats.py, test_random.py, test_advanced_index.py.
//
// Transcendental functions: Rust's f32/f64 methods (exp, ln, sin, cos, tanh, powf, ln_1p) lower
// to the platform libm; this file calls the same glibc functions. Their last-bit behaviour is
// glibc's, so bit-level parity with a Rust build on another libm is unpinned; the golden vectors
// pin them to the reference's own tolerances.
//
// Build: g++ -O2 -std=c++17 -ffp-contract=off -fno-fast-math (see oracle/Makefile). Contraction
// must stay off: the reference never fuses a multiply and an add in these kernels.
#include <cmath>
#include <cstdint>
#include <cstring>
#include <string>
#include <vector>

#include "../homura_amd/host/cpu_backend.h"
#include "../include/homura_rocm.h"
#include "elements.hpp"

namespace orc {
namespace {

thread_local std::string g_error;

struct Panic {
    std::string message;
};

[[noreturn]] void panic(std::string m) { throw Panic{std::move(m)}; }

const char *dtype_name(int d) {
    static const char *names[] = {"bool", "u8", "i8", "i16", "i32", "i64", "f16", "bf16", "f32", "f64"};
    return d >= 0 && d < 10 ? names[d] : "?";
}

// ---- Plan (ref: src/backend/cpu/iter.rs:17-94) --------------------------------------------------

template <int N>
struct Dim {
    int64_t size;
    int64_t st[N];
};

template <int N>
struct Plan {
    std::vector<Dim<N>> dims;
    bool empty = false;

    Plan(int ndim, const int64_t *shape, const int64_t *const (&strides)[N]) {
        for (int i = 0; i < ndim; ++i) {
            if (shape[i] == 0) {
                empty = true;
                return;
            }
        }
        for (int i = 0; i < ndim; ++i) {
            int64_t size = shape[i];
            if (size == 1) continue;
            Dim<N> d;
            d.size = size;
            for (int k = 0; k < N; ++k) d.st[k] = strides[k][i];
            if (!dims.empty()) {
                Dim<N> &outer = dims.back();
                bool joins = true;
                for (int k = 0; k < N; ++k) {
                    // checked_mul of the reference: an overflowing product never merges.
                    unsigned __int128 p = static_cast<unsigned __int128>(static_cast<uint64_t>(d.st[k])) *
                                          static_cast<uint64_t>(size);
                    if (p != static_cast<unsigned __int128>(static_cast<uint64_t>(outer.st[k]))) joins = false;
                }
                if (joins) {
                    outer.size *= size;
                    for (int k = 0; k < N; ++k) outer.st[k] = d.st[k];
                    continue;
                }
            }
            dims.push_back(d);
        }
    }

    template <class F>
    void recurse(size_t level, const int64_t (&base)[N], F &f) const {
        const Dim<N> &d = dims[level];
        int64_t off[N];
        for (int k = 0; k < N; ++k) off[k] = base[k];
        if (level + 1 == dims.size()) {
            for (int64_t i = 0; i < d.size; ++i) {
                f(off);
                for (int k = 0; k < N; ++k) off[k] += d.st[k];
            }
        } else {
            for (int64_t i = 0; i < d.size; ++i) {
                recurse(level + 1, off, f);
                for (int k = 0; k < N; ++k) off[k] += d.st[k];
            }
        }
    }

    // Calls f(offsets) for every element in row-major order.
    template <class F>
    void for_each(const int64_t (&base)[N], F f) const {
        if (empty) return;
        if (dims.empty()) {
            f(base);
        } else {
            recurse(0, base, f);
        }
    }
};

void check_shape(const hcb_tensor &out, const hcb_tensor &in) {
    bool same = out.ndim == in.ndim;
    for (int i = 0; same && i < out.ndim; ++i) same = out.shape[i] == in.shape[i];
    if (!same) panic("kernel operands must have the same shape");
}

int64_t num_elements(const hcb_tensor &t) {
    int64_t n = 1;
    for (int i = 0; i < t.ndim; ++i) n *= t.shape[i];
    return n;
}

bool is_contiguous(const hcb_tensor &t) {
    // ref: src/shape.rs:586-601 -- size-1 dimensions may have any stride; empty is contiguous.
    if (num_elements(t) == 0) return true;
    int64_t expect = 1;
    for (int i = t.ndim - 1; i >= 0; --i) {
        if (t.shape[i] != 1 && t.strides[i] != expect) return false;
        expect *= t.shape[i];
    }
    return true;
}

template <class T>
T *base(const hcb_tensor &t) {
    if (t.dtype != El<T>::code) panic("kernel instantiated for the wrong dtype");
    return static_cast<T *>(t.data);
}

// ---- map0..map3 (ref: src/backend/cpu/mod.rs:184-261) -----------------------------------------

template <class O, class F>
void map0(const hcb_tensor &out, F f) {
    O *po = base<O>(out);
    const int64_t *const st[1] = {out.strides};
    Plan<1> plan(out.ndim, out.shape, st);
    const int64_t b[1] = {out.offset};
    plan.for_each(b, [&](const int64_t(&o)[1]) { po[o[0]] = f(); });
}

template <class A, class O, class F>
void map1(const hcb_tensor &out, const hcb_tensor &a, F f) {
    check_shape(out, a);
    O *po = base<O>(out);
    const A *pa = base<A>(a);
    const int64_t *const st[2] = {out.strides, a.strides};
    Plan<2> plan(out.ndim, out.shape, st);
    const int64_t b[2] = {out.offset, a.offset};
    plan.for_each(b, [&](const int64_t(&o)[2]) { po[o[0]] = f(pa[o[1]]); });
}

template <class A, class B, class O, class F>
void map2(const hcb_tensor &out, const hcb_tensor &a, const hcb_tensor &b, F f) {
    check_shape(out, a);
    check_shape(out, b);
    O *po = base<O>(out);
    const A *pa = base<A>(a);
    const B *pb = base<B>(b);
    const int64_t *const st[3] = {out.strides, a.strides, b.strides};
    Plan<3> plan(out.ndim, out.shape, st);
    const int64_t bs[3] = {out.offset, a.offset, b.offset};
    plan.for_each(bs, [&](const int64_t(&o)[3]) { po[o[0]] = f(pa[o[1]], pb[o[2]]); });
}

template <class A, class B, class C, class O, class F>
void map3(const hcb_tensor &out, const hcb_tensor &a, const hcb_tensor &b, const hcb_tensor &c, F f) {
    check_shape(out, a);
    check_shape(out, b);
    check_shape(out, c);
    O *po = base<O>(out);
    const A *pa = base<A>(a);
    const B *pb = base<B>(b);
    const C *pc = base<C>(c);
    const int64_t *const st[4] = {out.strides, a.strides, b.strides, c.strides};
    Plan<4> plan(out.ndim, out.shape, st);
    const int64_t bs[4] = {out.offset, a.offset, b.offset, c.offset};
    plan.for_each(bs, [&](const int64_t(&o)[4]) { po[o[0]] = f(pa[o[1]], pb[o[2]], pc[o[3]]); });
}

// ---- dtype dispatch (ref: src/backend/cpu/mod.rs:66-168) --------------------------------------

template <class T>
struct Type {
    using type = T;
};

template <class F>
void dispatch_all(int dtype, F f) {
    switch (dtype) {
        case HMR_BOOL: f(Type<boolean>{}); break;
        case HMR_U8: f(Type<uint8_t>{}); break;
        case HMR_I8: f(Type<int8_t>{}); break;
        case HMR_I16: f(Type<int16_t>{}); break;
        case HMR_I32: f(Type<int32_t>{}); break;
        case HMR_I64: f(Type<int64_t>{}); break;
        case HMR_F16: f(Type<f16>{}); break;
        case HMR_BF16: f(Type<bf16>{}); break;
        case HMR_F32: f(Type<float>{}); break;
        case HMR_F64: f(Type<double>{}); break;
        default: panic("invalid dtype");
    }
}

template <class F>
void dispatch_float(int dtype, F f) {
    switch (dtype) {
        case HMR_F16: f(Type<f16>{}); break;
        case HMR_BF16: f(Type<bf16>{}); break;
        case HMR_F32: f(Type<float>{}); break;
        case HMR_F64: f(Type<double>{}); break;
        default: panic(std::string("expected a floating point dtype, got ") + dtype_name(dtype));
    }
}

template <class F>
void dispatch_int(int dtype, F f) {
    switch (dtype) {
        case HMR_U8: f(Type<uint8_t>{}); break;
        case HMR_I8: f(Type<int8_t>{}); break;
        case HMR_I16: f(Type<int16_t>{}); break;
        case HMR_I32: f(Type<int32_t>{}); break;
        case HMR_I64: f(Type<int64_t>{}); break;
        default: panic(std::string("expected an integer dtype, got ") + dtype_name(dtype));
    }
}

bool is_integral(int d) { return d >= HMR_U8 && d <= HMR_I64; }
bool is_float(int d) { return d >= HMR_F16 && d <= HMR_F64; }

// ---- wrapping integer arithmetic (ref: src/backend/cpu/num.rs:109-187) -------------------------

template <class T>
T wadd(T a, T b) {
    using U = std::make_unsigned_t<T>;
    return bit_cast<T>(static_cast<U>(static_cast<U>(a) + static_cast<U>(b)));
}
template <class T>
T wsub(T a, T b) {
    using U = std::make_unsigned_t<T>;
    return bit_cast<T>(static_cast<U>(static_cast<U>(a) - static_cast<U>(b)));
}
template <class T>
T wmul(T a, T b) {
    // Widen so that the promoted product of two u16-sized values cannot overflow `int`.
    using U = std::make_unsigned_t<T>;
    uint64_t p = static_cast<uint64_t>(static_cast<U>(a)) * static_cast<uint64_t>(static_cast<U>(b));
    return bit_cast<T>(static_cast<U>(p));
}
template <class T>
T wneg(T a) {
    return wsub<T>(T(0), a);
}
template <class T>
T wabs(T a) {
    if constexpr (std::is_unsigned_v<T>) return a;
    else return a < 0 ? wneg(a) : a;
}

template <class T>
T int_pow(T b, T exp) {
    int64_t e = static_cast<int64_t>(exp);
    if (e < 0) {
        int64_t bv = static_cast<int64_t>(b);
        if (bv == 1) return T(1);
        if (bv == -1) return e % 2 == 0 ? T(1) : b;
        return T(0);
    }
    T result = 1;
    uint64_t k = static_cast<uint64_t>(e);
    while (k > 0) {
        if (k & 1) result = wmul(result, b);
        b = wmul(b, b);
        k >>= 1;
    }
    return result;
}

// ---- erf (ref: src/backend/cpu/num.rs:189-219) -------------------------------------------------

double erf64(double x) {
    if (x != x) return x;
    double ax = std::fabs(x);
    double r;
    if (ax < 1.5) {
        double x2 = ax * ax;
        double term = ax;
        double sum = ax;
        double n = 0.0;
        while (term > 1e-17 * sum) {
            n += 1.0;
            term *= 2.0 * x2 / (2.0 * n + 1.0);
            sum += term;
        }
        r = 1.1283791670955125738961589031215452 /* FRAC_2_SQRT_PI */ * std::exp(-x2) * sum;
    } else if (ax < 6.0) {
        double f = ax;
        for (int k = 80; k >= 1; --k) f = ax + (static_cast<double>(k) * 0.5) / f;
        r = 1.0 - std::exp(-ax * ax) / (std::sqrt(3.14159265358979323846264338327950288) * f);
    } else {
        r = 1.0;
    }
    return std::copysign(r, x);
}

inline float erf_c(float x) { return static_cast<float>(erf64(static_cast<double>(x))); }
inline double erf_c(double x) { return erf64(x); }

template <class C>
C of(double v) {
    return static_cast<C>(v);
}

// ---- copy, fill (ref: src/backend/cpu/mod.rs:315-332) -----------------------------------------

template <class T>
T from_scalar(hcb_scalar s) {
    switch (s.kind) {
        case HCB_SCALAR_BOOL: return El<T>::from_bool(s.i != 0);
        case HCB_SCALAR_INT: return El<T>::from_i64(s.i);
        default: return El<T>::from_f64(s.f);
    }
}

void copy(const hcb_tensor &dst, const hcb_tensor &src) {
    if (src.dtype == dst.dtype) {
        dispatch_all(src.dtype, [&](auto t) {
            using T = typename decltype(t)::type;
            map1<T, T>(dst, src, [](T x) { return x; });
        });
    } else {
        dispatch_all(src.dtype, [&](auto s) {
            using S = typename decltype(s)::type;
            dispatch_all(dst.dtype, [&](auto d) {
                using D = typename decltype(d)::type;
                map1<S, D>(dst, src, [](S x) { return to_element<D, S>(x); });
            });
        });
    }
}

void fill(const hcb_tensor &dst, hcb_scalar value) {
    dispatch_all(dst.dtype, [&](auto t) {
        using T = typename decltype(t)::type;
        T v = from_scalar<T>(value);
        map0<T>(dst, [v]() { return v; });
    });
}

// ---- unary (ref: src/backend/cpu/mod.rs:336-407) ------------------------------------------------

template <class T>
void unary_float(int op, const hcb_tensor &out, const hcb_tensor &src) {
    using C = typename Fl<T>::C;
    auto run = [&](auto f) {
        map1<T, T>(out, src, [f](T v) {
            C x = Fl<T>::up(v);
            return Fl<T>::down(f(x));
        });
    };
    const C one = C(1), zero = C(0), half = of<C>(0.5);
    switch (op) {
        case HMR_UNARY_NEG: run([](C x) { return -x; }); break;
        case HMR_UNARY_ABS: run([](C x) { return std::fabs(x); }); break;
        case HMR_UNARY_RELU: run([=](C x) { return (x != x || x > zero) ? x : zero; }); break;
        case HMR_UNARY_SIGN:
            run([=](C x) { return x > zero ? one : (x < zero ? -one : zero); });
            break;
        case HMR_UNARY_EXP: run([](C x) { return std::exp(x); }); break;
        case HMR_UNARY_LOG: run([](C x) { return std::log(x); }); break;
        case HMR_UNARY_SQRT: run([](C x) { return std::sqrt(x); }); break;
        case HMR_UNARY_RSQRT: run([=](C x) { return one / std::sqrt(x); }); break;
        case HMR_UNARY_RECIPROCAL: run([=](C x) { return one / x; }); break;
        case HMR_UNARY_SIN: run([](C x) { return std::sin(x); }); break;
        case HMR_UNARY_COS: run([](C x) { return std::cos(x); }); break;
        case HMR_UNARY_ERF: run([](C x) { return erf_c(x); }); break;
        case HMR_UNARY_TANH: run([](C x) { return std::tanh(x); }); break;
        case HMR_UNARY_SIGMOID: run([=](C x) { return one / (one + std::exp(-x)); }); break;
        case HMR_UNARY_LOG_SIGMOID:
            run([=](C x) {
                C mn = (x != x || x < zero) ? x : zero;
                return mn - std::log1p(std::exp(-std::fabs(x)));
            });
            break;
        case HMR_UNARY_SILU: run([=](C x) { return x / (one + std::exp(-x)); }); break;
        case HMR_UNARY_GELU: {
            const C k = of<C>(0.70710678118654752440084436210484903 /* FRAC_1_SQRT_2 */);
            run([=](C x) { return half * x * (one + erf_c(x * k)); });
            break;
        }
        case HMR_UNARY_GELU_TANH: {
            const C k = of<C>(std::sqrt(2.0 / 3.14159265358979323846264338327950288));
            const C c = of<C>(0.044715);
            run([=](C x) { return half * x * (one + std::tanh(k * (x + c * x * x * x))); });
            break;
        }
        default: panic("invalid unary op");
    }
}

void unary(int op, const hcb_tensor &out, const hcb_tensor &src) {
    int dtype = src.dtype;
    if (op == HMR_UNARY_LOGICAL_NOT) {
        dispatch_all(dtype, [&](auto t) {
            using T = typename decltype(t)::type;
            map1<T, boolean>(out, src, [](T x) { return boolean{static_cast<uint8_t>(!El<T>::to_bool(x))}; });
        });
        return;
    }
    if (op == HMR_UNARY_SIGN && dtype == HMR_BOOL) {
        map1<boolean, boolean>(out, src, [](boolean x) { return x; });
        return;
    }
    bool int_op = op == HMR_UNARY_NEG || op == HMR_UNARY_ABS || op == HMR_UNARY_RELU || op == HMR_UNARY_SIGN;
    if (int_op && is_integral(dtype)) {
        dispatch_int(dtype, [&](auto t) {
            using T = typename decltype(t)::type;
            switch (op) {
                case HMR_UNARY_NEG: map1<T, T>(out, src, [](T x) { return wneg(x); }); break;
                case HMR_UNARY_ABS: map1<T, T>(out, src, [](T x) { return wabs(x); }); break;
                case HMR_UNARY_RELU: map1<T, T>(out, src, [](T x) { return x > T(0) ? x : T(0); }); break;
                default:
                    map1<T, T>(out, src, [](T x) { return x > T(0) ? T(1) : (x < T(0) ? wneg(T(1)) : T(0)); });
                    break;
            }
        });
        return;
    }
    dispatch_float(dtype, [&](auto t) {
        using T = typename decltype(t)::type;
        unary_float<T>(op, out, src);
    });
}

// ---- binary (ref: src/backend/cpu/mod.rs:409-466) -----------------------------------------------

const char *binary_name(int op) {
    static const char *names[] = {"Add", "Sub", "Mul", "Div", "Pow", "Maximum", "Minimum", "Greater",
                                  "GreaterEqual", "Less", "LessEqual", "Equal", "NotEqual",
                                  "LogicalAnd", "LogicalOr", "BitwiseAnd"};
    return op >= 0 && op < 16 ? names[op] : "?";
}

void binary(int op, const hcb_tensor &out, const hcb_tensor &a, const hcb_tensor &b) {
    int dtype = a.dtype;
    if (b.dtype != dtype) panic("binary operands have different dtypes");
    auto tf = [](bool v) { return boolean{static_cast<uint8_t>(v)}; };
    if (op >= HMR_BINARY_GREATER && op <= HMR_BINARY_NOT_EQUAL) {
        dispatch_all(dtype, [&](auto t) {
            using T = typename decltype(t)::type;
            switch (op) {
                case HMR_BINARY_GREATER: map2<T, T, boolean>(out, a, b, [=](T x, T y) { return tf(lt(y, x)); }); break;
                case HMR_BINARY_GREATER_EQUAL: map2<T, T, boolean>(out, a, b, [=](T x, T y) { return tf(le(y, x)); }); break;
                case HMR_BINARY_LESS: map2<T, T, boolean>(out, a, b, [=](T x, T y) { return tf(lt(x, y)); }); break;
                case HMR_BINARY_LESS_EQUAL: map2<T, T, boolean>(out, a, b, [=](T x, T y) { return tf(le(x, y)); }); break;
                case HMR_BINARY_EQUAL: map2<T, T, boolean>(out, a, b, [=](T x, T y) { return tf(eq(x, y)); }); break;
                default: map2<T, T, boolean>(out, a, b, [=](T x, T y) { return tf(!eq(x, y)); }); break;
            }
        });
        return;
    }
    if (op == HMR_BINARY_LOGICAL_AND) {
        map2<boolean, boolean, boolean>(out, a, b, [=](boolean x, boolean y) { return tf(x.v && y.v); });
        return;
    }
    if (op == HMR_BINARY_LOGICAL_OR) {
        map2<boolean, boolean, boolean>(out, a, b, [=](boolean x, boolean y) { return tf(x.v || y.v); });
        return;
    }
    if (op == HMR_BINARY_BITWISE_AND) {
        // Not in the reference (it has no bitwise op): two's-complement AND, logical and on bool.
        if (dtype == HMR_BOOL) {
            map2<boolean, boolean, boolean>(out, a, b, [=](boolean x, boolean y) { return tf(x.v && y.v); });
        } else if (is_integral(dtype)) {
            dispatch_int(dtype, [&](auto t) {
                using T = typename decltype(t)::type;
                map2<T, T, T>(out, a, b, [](T x, T y) { return static_cast<T>(x & y); });
            });
        } else {
            panic("BitwiseAnd is not supported for floating point tensors");
        }
        return;
    }
    if (dtype == HMR_BOOL) {
        switch (op) {
            case HMR_BINARY_ADD:
            case HMR_BINARY_MAXIMUM:
                map2<boolean, boolean, boolean>(out, a, b, [=](boolean x, boolean y) { return tf(x.v || y.v); });
                return;
            case HMR_BINARY_MUL:
            case HMR_BINARY_MINIMUM:
                map2<boolean, boolean, boolean>(out, a, b, [=](boolean x, boolean y) { return tf(x.v && y.v); });
                return;
            default: panic(std::string(binary_name(op)) + " is not supported for bool tensors");
        }
    }
    if (is_integral(dtype)) {
        dispatch_int(dtype, [&](auto t) {
            using T = typename decltype(t)::type;
            switch (op) {
                case HMR_BINARY_ADD: map2<T, T, T>(out, a, b, [](T x, T y) { return wadd(x, y); }); break;
                case HMR_BINARY_SUB: map2<T, T, T>(out, a, b, [](T x, T y) { return wsub(x, y); }); break;
                case HMR_BINARY_MUL: map2<T, T, T>(out, a, b, [](T x, T y) { return wmul(x, y); }); break;
                case HMR_BINARY_POW: map2<T, T, T>(out, a, b, [](T x, T y) { return int_pow(x, y); }); break;
                case HMR_BINARY_MAXIMUM: map2<T, T, T>(out, a, b, [](T x, T y) { return x > y ? x : y; }); break;
                case HMR_BINARY_MINIMUM: map2<T, T, T>(out, a, b, [](T x, T y) { return x < y ? x : y; }); break;
                default: panic(std::string(binary_name(op)) + " is not supported for integer tensors");
            }
        });
        return;
    }
    dispatch_float(dtype, [&](auto t) {
        using T = typename decltype(t)::type;
        using C = typename Fl<T>::C;
        auto run = [&](auto f) {
            map2<T, T, T>(out, a, b, [f](T u, T v) { return Fl<T>::down(f(Fl<T>::up(u), Fl<T>::up(v))); });
        };
        switch (op) {
            case HMR_BINARY_ADD: run([](C x, C y) { return x + y; }); break;
            case HMR_BINARY_SUB: run([](C x, C y) { return x - y; }); break;
            case HMR_BINARY_MUL: run([](C x, C y) { return x * y; }); break;
            case HMR_BINARY_DIV: run([](C x, C y) { return x / y; }); break;
            case HMR_BINARY_POW: run([](C x, C y) { return std::pow(x, y); }); break;
            case HMR_BINARY_MAXIMUM: run([](C x, C y) { return (x != x || x > y) ? x : y; }); break;
            case HMR_BINARY_MINIMUM: run([](C x, C y) { return (x != x || x < y) ? x : y; }); break;
            default: panic("invalid binary op");
        }
    });
}

// A zero-dimensional tensor of `dtype` holding `value`, broadcast to `like`'s shape.
struct Constant {
    alignas(8) unsigned char storage[8];
    std::vector<int64_t> zeros;
    hcb_tensor view;
    Constant(int dtype, hcb_scalar value, const hcb_tensor &like) : zeros(like.ndim > 0 ? like.ndim : 1, 0) {
        std::memset(storage, 0, sizeof storage);
        hcb_tensor cell{storage, 0, dtype, 0, nullptr, nullptr};
        fill(cell, value);
        view = hcb_tensor{storage, 0, dtype, like.ndim, like.shape, zeros.data()};
    }
};

// ref: src/backend/cpu/mod.rs:468-485
void binary_constant(int op, const hcb_tensor &out, const hcb_tensor &a, hcb_scalar value, bool constant_first) {
    Constant c(a.dtype, value, a);
    if (constant_first) binary(op, out, c.view, a);
    else binary(op, out, a, c.view);
}

// ref: src/backend/cpu/mod.rs:487-507
void binary_scalar(int op, const hcb_tensor &out, const hcb_tensor &a, double s, bool scalar_first) {
    dispatch_float(a.dtype, [&](auto t) {
        using T = typename decltype(t)::type;
        using C = typename Fl<T>::C;
        C sc = of<C>(s);
        if (op == HMR_BINARY_MUL) {
            map1<T, T>(out, a, [sc](T x) { return Fl<T>::down(Fl<T>::up(x) * sc); });
        } else if (op == HMR_BINARY_DIV && !scalar_first) {
            map1<T, T>(out, a, [sc](T x) { return Fl<T>::down(Fl<T>::up(x) / sc); });
        } else if (op == HMR_BINARY_DIV) {
            map1<T, T>(out, a, [sc](T x) { return Fl<T>::down(sc / Fl<T>::up(x)); });
        } else {
            panic(std::string(binary_name(op)) + " rounds its scalar to the dtype");
        }
    });
}

// ---- where (ref: src/backend/cpu/mod.rs:571-600) ------------------------------------------------

void where_(const hcb_tensor &out, const hcb_tensor &cond, const hcb_tensor &x, const hcb_tensor &y) {
    dispatch_all(out.dtype, [&](auto t) {
        using T = typename decltype(t)::type;
        map3<boolean, T, T, T>(out, cond, x, y, [](boolean c, T a, T b) { return c.v ? a : b; });
    });
}

void where_constant(const hcb_tensor &out, const hcb_tensor &cond, const hcb_tensor *x, hcb_scalar xv,
                    const hcb_tensor *y, hcb_scalar yv) {
    Constant cx(out.dtype, xv, out), cy(out.dtype, yv, out);
    where_(out, cond, x ? *x : cx.view, y ? *y : cy.view);
}

// ---- the optimizers' fused steps (ref: src/backend/cpu/mod.rs:509-569) -------------------------
//
// `kind`: 0 ScaledAdd(alpha), 1 Lerp(weight), 2 Addcmul(value), 3 Addcdiv(value); `c` only for 2
// and 3. Each element is computed in the computation type and rounded to the dtype once; mul_add
// is a true fused multiply-add (std::fma).
void fused(int kind, double scalar, const hcb_tensor &out, const hcb_tensor &a, const hcb_tensor &b,
           const hcb_tensor *c) {
    dispatch_float(out.dtype, [&](auto t) {
        using T = typename decltype(t)::type;
        using C = typename Fl<T>::C;
        auto mul_add = [](C x, C y, C z) { return static_cast<C>(std::fma(x, y, z)); };
        switch (kind) {
            case 0: {
                const C alpha = Fl<T>::up(Fl<T>::down(of<C>(scalar)));  // alpha rounded to the dtype first
                map2<T, T, T>(out, a, b, [=](T x, T y) { return Fl<T>::down(mul_add(Fl<T>::up(y), alpha, Fl<T>::up(x))); });
                break;
            }
            case 1: {
                const C weight = of<C>(scalar);
                const bool small = std::fabs(weight) < of<C>(0.5);
                const C coeff = small ? weight : weight - of<C>(1.0);
                map2<T, T, T>(out, a, b, [=](T x, T y) {
                    const C xc = Fl<T>::up(x), yc = Fl<T>::up(y);
                    return Fl<T>::down(mul_add(coeff, yc - xc, small ? xc : yc));
                });
                break;
            }
            case 2: {
                if (!c) panic("addcmul has three operands");
                const C value = of<C>(scalar);
                map3<T, T, T, T>(out, a, b, *c, [=](T x, T y, T z) {
                    return Fl<T>::down(mul_add(value * Fl<T>::up(y), Fl<T>::up(z), Fl<T>::up(x)));
                });
                break;
            }
            case 3: {
                if (!c) panic("addcdiv has three operands");
                const C value = of<C>(scalar);
                map3<T, T, T, T>(out, a, b, *c, [=](T x, T y, T z) {
                    return Fl<T>::down(Fl<T>::up(x) + value * Fl<T>::up(y) / Fl<T>::up(z));
                });
                break;
            }
            default: panic("unknown fused step");
        }
    });
}

// ---- triangle, flip (ref: src/backend/cpu/misc.rs:347-411) ---------------------------------------

void triangle(const hcb_tensor &out, const hcb_tensor &src, int64_t diagonal, bool upper) {
    check_shape(out, src);
    const int nd = src.ndim;
    if (nd < 2) panic("triangle needs two dimensions");
    if (num_elements(src) == 0) return;
    const int64_t rows = src.shape[nd - 2], cols = src.shape[nd - 1];
    dispatch_all(src.dtype, [&](auto t) {
        using T = typename decltype(t)::type;
        T *po = base<T>(out);
        const T *ps = base<T>(src);
        const int64_t *const st[2] = {out.strides, src.strides};
        Plan<2> batches(nd - 2, src.shape, st);
        const int64_t b[2] = {out.offset, src.offset};
        const int64_t ro = out.strides[nd - 2], co = out.strides[nd - 1];
        const int64_t rs = src.strides[nd - 2], cs = src.strides[nd - 1];
        batches.for_each(b, [&](const int64_t(&o)[2]) {
            for (int64_t r = 0; r < rows; ++r) {
                for (int64_t c = 0; c < cols; ++c) {
                    const int64_t d = c - r;
                    const bool keep = upper ? d >= diagonal : d <= diagonal;
                    po[o[0] + r * ro + c * co] = keep ? ps[o[1] + r * rs + c * cs] : T{};
                }
            }
        });
    });
}

// `out` is contiguous; `mask[d]` reverses dimension d.
void flip(const hcb_tensor &out, const hcb_tensor &src, const uint8_t *mask) {
    check_shape(out, src);
    const int64_t n = num_elements(src);
    const int nd = src.ndim;
    dispatch_all(src.dtype, [&](auto t) {
        using T = typename decltype(t)::type;
        T *po = base<T>(out);
        const T *ps = base<T>(src);
        std::vector<int64_t> idx(static_cast<size_t>(nd), 0);
        for (int64_t linear = 0; linear < n; ++linear) {
            int64_t off = src.offset;
            for (int d = 0; d < nd; ++d) {
                const int64_t i = mask[d] ? src.shape[d] - 1 - idx[d] : idx[d];
                off += i * src.strides[d];
            }
            po[out.offset + linear] = ps[off];
            for (int d = nd - 1; d >= 0; --d) {
                if (++idx[d] < src.shape[d]) break;
                idx[d] = 0;
            }
        }
    });
}

// ---- addr (ref: src/backend/cpu/linalg.rs:224-388) ----------------------------------------------
//
// out[i][j] = beta * input[i][j] + alpha * v1[i] * v2[j] for out [n, m], v1 [n], v2 [m] and an input
// viewed as [n, m] (read only when beta isn't zero), every step rounded to the dtype:
//   floats  a = alpha * v1[i] (skipped for alpha == 1), p = a * v2[j], c = beta * input (skipped for
//           beta == 1), out = c + p; alpha and beta in the computation type;
//   ints    wrapping i64: p = v1[i] * v2[j], times alpha unless 1, plus input (times beta unless 1);
//   bools   (input if beta) or (v1[i] and alpha and v2[j]).
template <class T, class Row, class Write>
void outer(const hcb_tensor &out, const hcb_tensor &v1, const hcb_tensor &v2, const hcb_tensor *input, Row row,
           Write write) {
    const int64_t n = v1.shape[0], m = v2.shape[0];
    if (out.ndim != 2 || out.shape[0] != n || out.shape[1] != m) panic("addr: the output isn't [n, m]");
    if (n == 0 || m == 0) return;
    if (input && (input->ndim != 2 || input->shape[0] != n || input->shape[1] != m)) panic("addr: the input isn't [n, m]");
    T *po = base<T>(out);
    const T *p1 = base<T>(v1), *p2 = base<T>(v2), *pc = input ? base<T>(*input) : nullptr;
    for (int64_t i = 0; i < n; ++i) {
        const T a = row(p1[v1.offset + i * v1.strides[0]]);
        for (int64_t j = 0; j < m; ++j) {
            const T y = p2[v2.offset + j * v2.strides[0]];
            const T *c = pc ? &pc[input->offset + i * input->strides[0] + j * input->strides[1]] : nullptr;
            po[out.offset + i * out.strides[0] + j * out.strides[1]] = write(a, y, c);
        }
    }
}

void addr(const hcb_tensor &out, const hcb_tensor &v1, const hcb_tensor &v2, const hcb_tensor &input, hcb_scalar alpha_s,
          hcb_scalar beta_s) {
    const int dtype = v1.dtype;
    auto f64_of = [](hcb_scalar s) { return s.kind == HCB_SCALAR_FLOAT ? s.f : static_cast<double>(s.i); };
    auto i64_of = [](hcb_scalar s) { return s.kind == HCB_SCALAR_FLOAT ? El<int64_t>::from_f64(s.f) : s.i; };
    auto bool_of = [](hcb_scalar s) { return s.kind == HCB_SCALAR_FLOAT ? s.f != 0.0 : s.i != 0; };
    if (is_float(dtype)) {
        dispatch_float(dtype, [&](auto t) {
            using T = typename decltype(t)::type;
            using C = typename Fl<T>::C;
            const C alpha = of<C>(f64_of(alpha_s)), beta = of<C>(f64_of(beta_s));
            outer<T>(
                out, v1, v2, beta != C(0) ? &input : nullptr,
                [=](T x) { return alpha == C(1) ? x : Fl<T>::down(Fl<T>::up(x) * alpha); },
                [=](T a, T y, const T *c) {
                    const T p = Fl<T>::down(Fl<T>::up(a) * Fl<T>::up(y));
                    if (!c) return p;
                    const T scaled = beta == C(1) ? *c : Fl<T>::down(Fl<T>::up(*c) * beta);
                    return Fl<T>::down(Fl<T>::up(scaled) + Fl<T>::up(p));
                });
        });
    } else if (is_integral(dtype)) {
        dispatch_int(dtype, [&](auto t) {
            using T = typename decltype(t)::type;
            const int64_t alpha = i64_of(alpha_s), beta = i64_of(beta_s);
            outer<T>(
                out, v1, v2, beta != 0 ? &input : nullptr, [](T x) { return x; },
                [=](T a, T y, const T *c) {
                    int64_t p = wmul<int64_t>(El<T>::to_i64(a), El<T>::to_i64(y));
                    if (alpha != 1) p = wmul<int64_t>(p, alpha);
                    if (!c) return El<T>::from_i64(p);
                    const int64_t ci = El<T>::to_i64(*c);
                    return El<T>::from_i64(wadd<int64_t>(beta == 1 ? ci : wmul<int64_t>(ci, beta), p));
                });
        });
    } else {
        const bool alpha = bool_of(alpha_s), beta = bool_of(beta_s);
        outer<boolean>(
            out, v1, v2, beta ? &input : nullptr, [=](boolean x) { return boolean{static_cast<uint8_t>(x.v && alpha)}; },
            [](boolean a, boolean y, const boolean *c) {
                return boolean{static_cast<uint8_t>((c && c->v) || (a.v && y.v))};
            });
    }
}

// ---- reductions (ref: src/backend/cpu/reduce.rs:10-225) ----------------------------------------

struct Split {
    std::vector<int64_t> kept_shape, kept_strides, red_shape, red_strides;
    Split(const hcb_tensor &src, const uint8_t *mask) {
        bool empty = num_elements(src) == 0;  // walk_strides: an empty source is walked with zeros
        for (int i = 0; i < src.ndim; ++i) {
            int64_t stride = empty ? 0 : src.strides[i];
            if (mask[i]) {
                red_shape.push_back(src.shape[i]);
                red_strides.push_back(stride);
            } else {
                kept_shape.push_back(src.shape[i]);
                kept_strides.push_back(stride);
            }
        }
    }
};

std::vector<int64_t> contiguous_strides(const std::vector<int64_t> &shape) {
    std::vector<int64_t> st(shape.size());
    int64_t s = 1;
    for (int i = static_cast<int>(shape.size()) - 1; i >= 0; --i) {
        st[i] = s;
        s *= shape[i];
    }
    return st;
}

int64_t product(const std::vector<int64_t> &v) {
    int64_t n = 1;
    for (int64_t x : v) n *= x;
    return n;
}

template <class S, class O, class A, class Step, class Finish>
void fold(const hcb_tensor &out, const hcb_tensor &src, const uint8_t *mask, A init, Step step, Finish finish) {
    Split s(src, mask);
    int64_t count = product(s.red_shape);
    std::vector<int64_t> out_strides = contiguous_strides(s.kept_shape);
    if (!is_contiguous(out)) panic("assertion failed: out.layout.is_contiguous()");
    if (num_elements(out) != product(s.kept_shape)) panic("assertion failed: output size");
    O *po = base<O>(out);
    const S *ps = base<S>(src);
    const int64_t *const ost[2] = {out_strides.data(), s.kept_strides.data()};
    Plan<2> outer(static_cast<int>(s.kept_shape.size()), s.kept_shape.data(), ost);
    const int64_t *const ist[1] = {s.red_strides.data()};
    Plan<1> inner(static_cast<int>(s.red_shape.size()), s.red_shape.data(), ist);
    const int64_t b[2] = {out.offset, src.offset};
    outer.for_each(b, [&](const int64_t(&o)[2]) {
        A acc = init;
        const int64_t ib[1] = {o[1]};
        inner.for_each(ib, [&](const int64_t(&j)[1]) { acc = step(acc, ps[j[0]]); });
        po[o[0]] = finish(acc, count);
    });
}

template <class T>
struct Best {
    bool some;
    T v;
};

template <class T>
bool is_nan_el(T v) {
    return !eq(v, v);
}

// ref: src/backend/cpu/reduce.rs:75-86
template <class T>
bool replaces(const Best<T> &acc, T x, bool is_max) {
    if (!acc.some) return true;
    if (is_nan_el(acc.v)) return false;
    return is_nan_el(x) || (is_max ? lt(acc.v, x) : lt(x, acc.v));
}

void reduce(int op, const hcb_tensor &out, const hcb_tensor &src, const uint8_t *mask) {
    int dtype = src.dtype;
    bool sum_like = op == HMR_REDUCE_SUM || op == HMR_REDUCE_PROD || op == HMR_REDUCE_MEAN;
    if (sum_like && is_float(dtype)) {
        dispatch_float(dtype, [&](auto t) {
            using T = typename decltype(t)::type;
            if (op == HMR_REDUCE_SUM) {
                fold<T, T, double>(out, src, mask, 0.0, [](double a, T x) { return a + El<T>::to_f64(x); },
                                   [](double a, int64_t) { return El<T>::from_f64(a); });
            } else if (op == HMR_REDUCE_PROD) {
                fold<T, T, double>(out, src, mask, 1.0, [](double a, T x) { return a * El<T>::to_f64(x); },
                                   [](double a, int64_t) { return El<T>::from_f64(a); });
            } else {
                fold<T, T, double>(out, src, mask, 0.0, [](double a, T x) { return a + El<T>::to_f64(x); },
                                   [](double a, int64_t n) { return El<T>::from_f64(a / static_cast<double>(n)); });
            }
        });
        return;
    }
    if (op == HMR_REDUCE_SUM || op == HMR_REDUCE_PROD) {
        if (out.dtype != HMR_I64) panic("assertion failed: out.dtype == I64");
        dispatch_all(dtype, [&](auto t) {
            using T = typename decltype(t)::type;
            if (op == HMR_REDUCE_SUM) {
                fold<T, int64_t, int64_t>(out, src, mask, 0,
                                          [](int64_t a, T x) { return wadd<int64_t>(a, El<T>::to_i64(x)); },
                                          [](int64_t a, int64_t) { return a; });
            } else {
                fold<T, int64_t, int64_t>(out, src, mask, 1,
                                          [](int64_t a, T x) { return wmul<int64_t>(a, El<T>::to_i64(x)); },
                                          [](int64_t a, int64_t) { return a; });
            }
        });
        return;
    }
    if (op == HMR_REDUCE_MEAN) panic(std::string("mean requires a floating point input, got ") + dtype_name(dtype));
    if (op == HMR_REDUCE_MAX || op == HMR_REDUCE_MIN) {
        bool is_max = op == HMR_REDUCE_MAX;
        dispatch_all(dtype, [&](auto t) {
            using T = typename decltype(t)::type;
            fold<T, T, Best<T>>(
                out, src, mask, Best<T>{false, T{}},
                [is_max](Best<T> a, T x) { return replaces(a, x, is_max) ? Best<T>{true, x} : a; },
                [](Best<T> a, int64_t) {
                    if (!a.some) panic("reduction over an empty dimension");
                    return a.v;
                });
        });
        return;
    }
    if (op == HMR_REDUCE_ALL || op == HMR_REDUCE_ANY) {
        bool all = op == HMR_REDUCE_ALL;
        dispatch_all(dtype, [&](auto t) {
            using T = typename decltype(t)::type;
            auto step = [all](bool a, T x) { return all ? (a && El<T>::to_bool(x)) : (a || El<T>::to_bool(x)); };
            if (out.dtype == HMR_U8) {
                fold<T, uint8_t, bool>(out, src, mask, all, step, [](bool a, int64_t) { return static_cast<uint8_t>(a); });
            } else {
                fold<T, boolean, bool>(out, src, mask, all, step,
                                       [](bool a, int64_t) { return boolean{static_cast<uint8_t>(a)}; });
            }
        });
        return;
    }
    panic("invalid reduce op");
}

// ref: src/backend/cpu/reduce.rs:133-170
void var(const hcb_tensor &out, const hcb_tensor &src, const uint8_t *mask, double correction, bool take_sqrt) {
    dispatch_float(src.dtype, [&](auto t) {
        using T = typename decltype(t)::type;
        Split s(src, mask);
        int64_t count = product(s.red_shape);
        std::vector<int64_t> out_strides = contiguous_strides(s.kept_shape);
        if (!is_contiguous(out)) panic("assertion failed: out.layout.is_contiguous()");
        T *po = base<T>(out);
        const T *ps = base<T>(src);
        const int64_t *const ost[2] = {out_strides.data(), s.kept_strides.data()};
        Plan<2> outer(static_cast<int>(s.kept_shape.size()), s.kept_shape.data(), ost);
        const int64_t *const ist[1] = {s.red_strides.data()};
        Plan<1> inner(static_cast<int>(s.red_shape.size()), s.red_shape.data(), ist);
        double divisor = std::fmax(static_cast<double>(count) - correction, 0.0);
        const int64_t b[2] = {out.offset, src.offset};
        outer.for_each(b, [&](const int64_t(&o)[2]) {
            const int64_t ib[1] = {o[1]};
            double sum = 0.0;
            inner.for_each(ib, [&](const int64_t(&j)[1]) { sum += El<T>::to_f64(ps[j[0]]); });
            double mean = sum / static_cast<double>(count);
            double sq = 0.0;
            inner.for_each(ib, [&](const int64_t(&j)[1]) {
                double d = El<T>::to_f64(ps[j[0]]) - mean;
                sq += d * d;
            });
            double v = count == 0 ? std::numeric_limits<double>::quiet_NaN() : sq / divisor;
            po[o[0]] = El<T>::from_f64(take_sqrt ? std::sqrt(v) : v);
        });
    });
}

// ref: src/backend/cpu/reduce.rs:172-225
void arg_reduce(const hcb_tensor *values, const hcb_tensor &indices, const hcb_tensor &src, int dim, bool is_max) {
    int64_t n = 1, stride = 0;
    if (src.ndim > 0) {
        n = src.shape[dim];
        stride = src.strides[dim];
    }
    if (n <= 0) panic("cannot compute the arg reduction of an empty dimension");
    std::vector<uint8_t> mask(src.ndim, 0);
    if (src.ndim > 0) mask[dim] = 1;
    Split s(src, mask.data());
    std::vector<int64_t> out_strides = contiguous_strides(s.kept_shape);
    dispatch_all(src.dtype, [&](auto t) {
        using T = typename decltype(t)::type;
        const T *ps = base<T>(src);
        int64_t *pi = base<int64_t>(indices);
        T *pv = values ? base<T>(*values) : nullptr;
        const int64_t *const ost[2] = {out_strides.data(), s.kept_strides.data()};
        Plan<2> outer(static_cast<int>(s.kept_shape.size()), s.kept_shape.data(), ost);
        const int64_t b[2] = {0, src.offset};
        outer.for_each(b, [&](const int64_t(&o)[2]) {
            Best<T> best{false, T{}};
            int64_t best_index = 0;
            for (int64_t k = 0; k < n; ++k) {
                T x = ps[o[1] + k * stride];
                if (replaces(best, x, is_max)) {
                    best = Best<T>{true, x};
                    best_index = k;
                }
            }
            pi[indices.offset + o[0]] = best_index;
            if (pv) pv[values->offset + o[0]] = best.v;
        });
    });
}

// ---- softmax (ref: src/backend/cpu/misc.rs:13-51) ----------------------------------------------

void softmax(const hcb_tensor &out, const hcb_tensor &src, int dim, bool log) {
    check_shape(out, src);
    if (num_elements(src) == 0) return;
    bool scalar = src.ndim == 0;
    int64_t n = 1, si = 0, so = 0;
    std::vector<int64_t> kshape, ks_strides, ko_strides;
    if (!scalar) {
        n = src.shape[dim];
        si = src.strides[dim];
        so = out.strides[dim];
        for (int i = 0; i < src.ndim; ++i) {
            if (i == dim) continue;
            kshape.push_back(src.shape[i]);
            ks_strides.push_back(src.strides[i]);
            ko_strides.push_back(out.strides[i]);
        }
    }
    dispatch_float(src.dtype, [&](auto t) {
        using T = typename decltype(t)::type;
        const T *ps = base<T>(src);
        T *po = base<T>(out);
        const int64_t *const st[2] = {ko_strides.data(), ks_strides.data()};
        Plan<2> outer(static_cast<int>(kshape.size()), kshape.data(), st);
        const int64_t b[2] = {out.offset, src.offset};
        outer.for_each(b, [&](const int64_t(&o)[2]) {
            auto x = [&](int64_t k) { return El<T>::to_f64(ps[o[1] + k * si]); };
            double mx = -std::numeric_limits<double>::infinity();
            for (int64_t k = 0; k < n; ++k) {
                double v = x(k);
                mx = v > mx ? v : mx;
            }
            double sum = 0.0;
            for (int64_t k = 0; k < n; ++k) sum += std::exp(x(k) - mx);
            double log_sum = std::log(sum);
            for (int64_t k = 0; k < n; ++k) {
                double v = log ? x(k) - mx - log_sum : std::exp(x(k) - mx) / sum;
                po[o[0] + k * so] = El<T>::from_f64(v);
            }
        });
    });
}

// ---- exclusive cumulative product (ref: src/backend/cpu/reduce.rs:227-324) -----------------------
//
// For each element, the product of the elements before it along `dim` (after it when `reverse`):
// accumulated one element at a time in the accumulation type of the dtype (f32 for F16 and BF16,
// f64 for F32 and F64), each output rounded from the accumulator, which itself is never rounded.
template <class T>
struct Accumulate {
    using A = float;
    static A widen(T x) { return Fl<T>::up(x); }
    static T narrow(A acc) { return Fl<T>::down(acc); }
};
template <>
struct Accumulate<float> {
    using A = double;
    static A widen(float x) { return static_cast<double>(x); }
    static float narrow(A acc) { return static_cast<float>(acc); }
};
template <>
struct Accumulate<double> {
    using A = double;
    static A widen(double x) { return x; }
    static double narrow(A acc) { return acc; }
};

void exclusive_cumprod(const hcb_tensor &out, const hcb_tensor &src, int dim, bool reverse) {
    check_shape(out, src);
    if (out.dtype != src.dtype) panic("exclusive_cumprod: the operands have different dtypes");
    if (num_elements(src) == 0) return;
    if (dim < 0 || dim >= src.ndim) panic("exclusive_cumprod: dimension out of range");
    const int64_t n = src.shape[dim], si = src.strides[dim], so = out.strides[dim];
    std::vector<int64_t> kshape, ks_strides, ko_strides;
    for (int i = 0; i < src.ndim; ++i) {
        if (i == dim) continue;
        kshape.push_back(src.shape[i]);
        ks_strides.push_back(src.strides[i]);
        ko_strides.push_back(out.strides[i]);
    }
    dispatch_float(src.dtype, [&](auto t) {
        using T = typename decltype(t)::type;
        using Acc = Accumulate<T>;
        const T *ps = base<T>(src);
        T *po = base<T>(out);
        const int64_t *const st[2] = {ko_strides.data(), ks_strides.data()};
        Plan<2> lines(static_cast<int>(kshape.size()), kshape.data(), st);
        const int64_t b[2] = {out.offset, src.offset};
        lines.for_each(b, [&](const int64_t(&o)[2]) {
            typename Acc::A acc = 1;
            for (int64_t k = 0; k < n; ++k) {
                const int64_t at = reverse ? n - 1 - k : k;
                po[o[0] + at * so] = Acc::narrow(acc);
                acc = acc * Acc::widen(ps[o[1] + at * si]);
            }
        });
    });
}

// ---- random sampling (ref: src/ops/random.rs:29-226) ---------------------------------------------
//
// Philox4x32-10: block n is the counter [n, n >> 32, 0, 0] under the key [seed, seed >> 32]. The
// caller reserves a call's blocks (from `offset` on) and advances its generator.
void philox(const uint32_t counter[4], const uint32_t key[2], uint32_t out[4]) {
    const uint64_t M0 = 0xD2511F53u, M1 = 0xCD9E8D57u;
    const uint32_t W0 = 0x9E3779B9u, W1 = 0xBB67AE85u;
    uint32_t c[4] = {counter[0], counter[1], counter[2], counter[3]};
    uint32_t k[2] = {key[0], key[1]};
    for (int round = 0; round < 10; ++round) {
        if (round > 0) {
            k[0] += W0;
            k[1] += W1;
        }
        const uint64_t p0 = M0 * c[0], p1 = M1 * c[2];
        const uint32_t n0 = static_cast<uint32_t>(p1 >> 32) ^ c[1] ^ k[0], n1 = static_cast<uint32_t>(p1);
        const uint32_t n2 = static_cast<uint32_t>(p0 >> 32) ^ c[3] ^ k[1], n3 = static_cast<uint32_t>(p0);
        c[0] = n0, c[1] = n1, c[2] = n2, c[3] = n3;
    }
    for (int i = 0; i < 4; ++i) out[i] = c[i];
}

struct Blocks {
    uint64_t seed, start;
    void operator()(uint64_t i, uint32_t out[4]) const {
        const uint64_t n = start + i;
        const uint32_t counter[4] = {static_cast<uint32_t>(n), static_cast<uint32_t>(n >> 32), 0, 0};
        const uint32_t key[2] = {static_cast<uint32_t>(seed), static_cast<uint32_t>(seed >> 32)};
        philox(counter, key, out);
    }
};

// A uniform f64 in [0, 1) from 53 random bits / from the top `bits` bits of x.
double unit_f64(uint32_t hi, uint32_t lo) {
    const uint64_t bits = (static_cast<uint64_t>(hi) << 21) ^ (static_cast<uint64_t>(lo) >> 11);
    return static_cast<double>(bits) * (1.0 / 9007199254740992.0);
}
double unit_bits(uint32_t x, int bits) { return static_cast<double>(x >> (32 - bits)) / static_cast<double>(uint64_t{1} << bits); }

int float_digits(int dtype) { return dtype == HMR_F16 ? 11 : dtype == HMR_BF16 ? 8 : dtype == HMR_F32 ? 24 : 53; }

void check_flat(const hcb_tensor &out) {
    int64_t expect = 1;
    for (int d = out.ndim - 1; d >= 0; --d) {
        if (out.shape[d] != 1 && out.strides[d] != expect) panic("random sampling writes a contiguous tensor");
        expect *= out.shape[d];
    }
}

void random_uniform(const hcb_tensor &out, uint64_t seed, uint64_t offset, double from, double to) {
    check_flat(out);
    const int64_t n = num_elements(out);
    dispatch_float(out.dtype, [&](auto t) {
        using T = typename decltype(t)::type;
        T *po = base<T>(out) + out.offset;
        const int per_block = out.dtype == HMR_F64 ? 2 : 4;  // f64 uses two words per value
        const int bits = float_digits(out.dtype);
        const Blocks block{seed, offset};
        for (int64_t i = 0; i * per_block < n; ++i) {
            uint32_t b[4];
            block(static_cast<uint64_t>(i), b);
            for (int j = 0; j < per_block && i * per_block + j < n; ++j) {
                const double u = per_block == 2 ? unit_f64(b[2 * j], b[2 * j + 1]) : unit_bits(b[j], bits);
                const double x = from + u * (to - from);
                T v = El<T>::from_f64(x);
                // Rounding can reach the excluded upper bound, which maps to the lower one.
                if (from < to && El<T>::to_f64(v) >= to) v = El<T>::from_f64(from);
                po[i * per_block + j] = v;
            }
        }
    });
}

void random_normal(const hcb_tensor &out, uint64_t seed, uint64_t offset, double mean, double std) {
    check_flat(out);
    const int64_t n = num_elements(out);
    dispatch_float(out.dtype, [&](auto t) {
        using T = typename decltype(t)::type;
        T *po = base<T>(out) + out.offset;
        const Blocks block{seed, offset};
        for (int64_t i = 0; 2 * i < n; ++i) {  // Box-Muller: each block gives two normals
            uint32_t b[4];
            block(static_cast<uint64_t>(i), b);
            const double u1 = 1.0 - unit_f64(b[0], b[1]), u2 = unit_f64(b[2], b[3]);
            const double r = std::sqrt(-2.0 * std::log(u1));
            const double theta = 2.0 * 3.14159265358979323846 * u2;
            po[2 * i] = El<T>::from_f64(mean + std * r * std::cos(theta));
            if (2 * i + 1 < n) po[2 * i + 1] = El<T>::from_f64(mean + std * r * std::sin(theta));
        }
    });
}

// One batch of rejection sampling on 64-bit words (two per block: [w0 w1], then [w2 w3]): the words
// >= threshold become low + word % range and fill the I64 `out` until it is full. Returns how many
// words of the batch were accepted (which may exceed out's elements).
uint64_t random_int(const hcb_tensor &out, uint64_t seed, uint64_t offset, uint64_t blocks, int64_t low, uint64_t range,
                    uint64_t threshold) {
    check_flat(out);
    if (out.dtype != HMR_I64) panic("random integers are sampled into an I64 tensor");
    if (range == 0) panic("random_int: empty range");
    const uint64_t n = static_cast<uint64_t>(num_elements(out));
    int64_t *po = base<int64_t>(out) + out.offset;
    const Blocks block{seed, offset};
    uint64_t accepted = 0;
    for (uint64_t i = 0; i < blocks; ++i) {
        uint32_t b[4];
        block(i, b);
        const uint64_t words[2] = {(static_cast<uint64_t>(b[0]) << 32) | b[1], (static_cast<uint64_t>(b[2]) << 32) | b[3]};
        for (uint64_t w : words) {
            if (w < threshold) continue;
            if (accepted < n) po[accepted] = static_cast<int64_t>(static_cast<uint64_t>(low) + w % range);
            ++accepted;
        }
    }
    return accepted;
}

// ---- indexing (ref: src/backend/cpu/misc.rs:53-127, 213-345; src/backend/mod.rs:360-378) ----------
//
// `bounds`: 0 the positions are valid, 1 none may be negative, 2 negative ones count from the end.
// The first position out of range, in row-major order of the index, is the error.
std::vector<int64_t> positions(const hcb_tensor &index, int dim, int64_t size, int bounds) {
    std::vector<int64_t> out;
    const int64_t n = num_elements(index);
    out.reserve(static_cast<size_t>(n));
    const int64_t low = bounds == 2 ? -size : 0;
    auto take = [&](int64_t v) {
        if (bounds != 0 && !(v >= low && v < size)) {
            panic("index " + std::to_string(v) + " is out of bounds for dimension " + std::to_string(dim) + " with size " +
                  std::to_string(size));
        }
        out.push_back(v < 0 ? v + size : v);
    };
    const int64_t *const st[1] = {index.strides};
    Plan<1> plan(index.ndim, index.shape, st);
    const int64_t b[1] = {index.offset};
    if (index.dtype == HMR_I64) {
        const int64_t *p = base<int64_t>(index);
        plan.for_each(b, [&](const int64_t(&o)[1]) { take(p[o[0]]); });
    } else if (index.dtype == HMR_I32) {
        const int32_t *p = base<int32_t>(index);
        plan.for_each(b, [&](const int64_t(&o)[1]) { take(p[o[0]]); });
    } else {
        panic("an index tensor is I32 or I64");
    }
    return out;
}

// out = the slices of src along dim picked by the 1-D index (ref: misc.rs:74-105).
void index_select(const hcb_tensor &out, const hcb_tensor &src, int dim, const hcb_tensor &index, int bounds) {
    const std::vector<int64_t> picked = positions(index, dim, src.shape[dim], bounds);
    if (num_elements(out) == 0) return;
    std::vector<int64_t> shape, so, ss;
    for (int d = 0; d < out.ndim; ++d) {
        if (d == dim) continue;
        shape.push_back(out.shape[d]);
        so.push_back(out.strides[d]);
        ss.push_back(src.strides[d]);
    }
    dispatch_all(src.dtype, [&](auto t) {
        using T = typename decltype(t)::type;
        T *po = base<T>(out);
        const T *ps = base<T>(src);
        const int64_t *const st[2] = {so.data(), ss.data()};
        Plan<2> slice(static_cast<int>(shape.size()), shape.data(), st);
        for (size_t j = 0; j < picked.size(); ++j) {
            const int64_t b[2] = {out.offset + static_cast<int64_t>(j) * out.strides[dim], src.offset + picked[j] * src.strides[dim]};
            slice.for_each(b, [&](const int64_t(&o)[2]) { po[o[0]] = ps[o[1]]; });
        }
    });
}

// out[p] = src[.., index[p], ..] for every position p of the contiguous out, which has the index's shape
// (ref: misc.rs:313-345).
void gather(const hcb_tensor &out, const hcb_tensor &src, int dim, const hcb_tensor &index) {
    const std::vector<int64_t> picked = positions(index, dim, src.shape[dim], 1);
    if (picked.empty()) return;
    std::vector<int64_t> walk(src.strides, src.strides + src.ndim);
    walk[dim] = 0;  // the index value replaces the position along dim
    dispatch_all(src.dtype, [&](auto t) {
        using T = typename decltype(t)::type;
        T *po = base<T>(out);
        const T *ps = base<T>(src);
        const int64_t *const st[2] = {out.strides, walk.data()};
        Plan<2> plan(out.ndim, out.shape, st);
        const int64_t b[2] = {out.offset, src.offset};
        size_t k = 0;
        plan.for_each(b, [&](const int64_t(&o)[2]) { po[o[0]] = ps[o[1] + picked[k++] * src.strides[dim]]; });
    });
}

// out[o] += src[s] for the pairs `pairs` reports in order: each element of the contiguous out is
// accumulated in f64 (floats) or wrapping i64 (integers; an or for bools) and rounded once at the end
// (ref: misc.rs:213-252).
template <class Pairs>
void add_at(const hcb_tensor &out, const hcb_tensor &src, Pairs pairs) {
    const int64_t n = num_elements(out);
    if (n == 0) return;
    if (out.dtype != src.dtype) panic("add_at: the operands have different dtypes");
    dispatch_all(out.dtype, [&](auto t) {
        using T = typename decltype(t)::type;
        T *elements = base<T>(out) + out.offset;
        const T *ps = base<T>(src);
        if (is_float(out.dtype)) {
            std::vector<double> acc(static_cast<size_t>(n));
            for (int64_t i = 0; i < n; ++i) acc[i] = El<T>::to_f64(elements[i]);
            pairs([&](int64_t o, int64_t s) { acc[o] += El<T>::to_f64(ps[s]); });
            for (int64_t i = 0; i < n; ++i) elements[i] = El<T>::from_f64(acc[i]);
        } else {
            std::vector<int64_t> acc(static_cast<size_t>(n));
            for (int64_t i = 0; i < n; ++i) acc[i] = El<T>::to_i64(elements[i]);
            pairs([&](int64_t o, int64_t s) { acc[o] = wadd<int64_t>(acc[o], El<T>::to_i64(ps[s])); });
            for (int64_t i = 0; i < n; ++i) elements[i] = El<T>::from_i64(acc[i]);
        }
    });
}

std::vector<int64_t> contiguous_strides_of(const int64_t *shape, int ndim) {
    std::vector<int64_t> st(static_cast<size_t>(ndim), 1);
    for (int d = ndim - 2; d >= 0; --d) st[d] = st[d + 1] * shape[d + 1];
    return st;
}

// Adds slice i of src along dim into slice index[i] of the contiguous out (ref: misc.rs:254-290).
void index_add(const hcb_tensor &out, int dim, const hcb_tensor &index, const hcb_tensor &src, int bounds) {
    const std::vector<int64_t> picked = positions(index, dim, out.shape[dim], bounds);
    if (num_elements(src) == 0) return;
    const std::vector<int64_t> out_strides = contiguous_strides_of(out.shape, out.ndim);
    std::vector<int64_t> shape, so, ss;
    for (int d = 0; d < src.ndim; ++d) {
        if (d == dim) continue;
        shape.push_back(src.shape[d]);
        so.push_back(out_strides[d]);
        ss.push_back(src.strides[d]);
    }
    const int64_t *const st[2] = {so.data(), ss.data()};
    Plan<2> plan(static_cast<int>(shape.size()), shape.data(), st);
    add_at(out, src, [&](auto f) {
        for (size_t i = 0; i < picked.size(); ++i) {
            const int64_t b[2] = {picked[i] * out_strides[dim], src.offset + static_cast<int64_t>(i) * src.strides[dim]};
            plan.for_each(b, [&](const int64_t(&o)[2]) { f(o[0], o[1]); });
        }
    });
}

// out[.., index[p], ..] += src[p] for every position p of the index (ref: misc.rs:292-311).
void scatter_add(const hcb_tensor &out, int dim, const hcb_tensor &index, const hcb_tensor &src) {
    const std::vector<int64_t> picked = positions(index, dim, out.shape[dim], 1);
    if (picked.empty()) return;
    const std::vector<int64_t> out_strides = contiguous_strides_of(out.shape, out.ndim);
    std::vector<int64_t> walk = out_strides;
    walk[dim] = 0;
    const int64_t *const st[2] = {walk.data(), src.strides};
    Plan<2> plan(index.ndim, index.shape, st);
    add_at(out, src, [&](auto f) {
        size_t k = 0;
        const int64_t b[2] = {0, src.offset};
        plan.for_each(b, [&](const int64_t(&o)[2]) { f(o[0] + picked[k++] * out_strides[dim], o[1]); });
    });
}

// The elements of an I32 or I64 tensor in row-major order, as i64 (ref: misc.rs read_host::<i64>).
std::vector<int64_t> integers_of(const hcb_tensor &t) {
    std::vector<int64_t> out;
    out.reserve(static_cast<size_t>(num_elements(t)));
    const int64_t *const st[1] = {t.strides};
    Plan<1> plan(t.ndim, t.shape, st);
    const int64_t b[1] = {t.offset};
    if (t.dtype == HMR_I64) {
        const int64_t *p = base<int64_t>(t);
        plan.for_each(b, [&](const int64_t(&o)[1]) { out.push_back(p[o[0]]); });
    } else if (t.dtype == HMR_I32) {
        const int32_t *p = base<int32_t>(t);
        plan.for_each(b, [&](const int64_t(&o)[1]) { out.push_back(p[o[0]]); });
    } else {
        panic("an index tensor is I32 or I64");
    }
    return out;
}

// Copies slice i of src along dim into slice index[i] of out, in order, so that the last of repeated
// positions wins (ref: misc.rs:104-126). The positions are valid.
void index_overwrite(const hcb_tensor &out, int dim, const hcb_tensor &index, const hcb_tensor &src) {
    if (num_elements(src) == 0) return;
    const std::vector<int64_t> picked = positions(index, dim, out.shape[dim], 0);
    std::vector<int64_t> shape, so, ss;
    for (int d = 0; d < src.ndim; ++d) {
        if (d == dim) continue;
        shape.push_back(src.shape[d]);
        so.push_back(out.strides[d]);
        ss.push_back(src.strides[d]);
    }
    dispatch_all(src.dtype, [&](auto t) {
        using T = typename decltype(t)::type;
        T *po = base<T>(out);
        const T *ps = base<T>(src);
        const int64_t *const st[2] = {so.data(), ss.data()};
        Plan<2> slice(static_cast<int>(shape.size()), shape.data(), st);
        for (size_t i = 0; i < picked.size(); ++i) {
            const int64_t b[2] = {out.offset + picked[i] * out.strides[dim], src.offset + static_cast<int64_t>(i) * src.strides[dim]};
            slice.for_each(b, [&](const int64_t(&o)[2]) { po[o[0]] = ps[o[1]]; });
        }
    });
}

// The number of true elements of a BOOL mask and, with `out` (I64, contiguous, the mask's rank x that number),
// coordinate d of the k-th of them in row-major order at out[d][k] (ref: misc.rs:128-148).
int64_t mask_coordinates(const hcb_tensor &mask, const hcb_tensor *out) {
    if (mask.dtype != HMR_BOOL) panic("a mask is a BOOL tensor");
    const boolean *p = base<boolean>(mask);
    const int64_t *const st[1] = {mask.strides};
    Plan<1> plan(mask.ndim, mask.shape, st);
    const int64_t b[1] = {mask.offset};
    int64_t count = 0;
    plan.for_each(b, [&](const int64_t(&o)[1]) { count += p[o[0]].v != 0; });
    if (out == nullptr) return count;
    int64_t *po = base<int64_t>(*out) + out->offset;
    std::vector<int64_t> at(static_cast<size_t>(mask.ndim), 0);
    int64_t k = 0;
    plan.for_each(b, [&](const int64_t(&o)[1]) {
        if (p[o[0]].v != 0) {
            for (int d = 0; d < mask.ndim; ++d) po[d * count + k] = at[d];
            ++k;
        }
        for (int d = mask.ndim - 1; d >= 0; --d) {
            if (++at[d] < mask.shape[d]) break;
            at[d] = 0;
        }
    });
    return count;
}

// Checks each of the `n` indices, in order and each in row-major order, to lie in -size..size for its size
// in `sizes`; the first one out of range is reported as (bad_index, bad_value) and nothing is written.
// Otherwise (bad_index = -1), and with `out` (I64, contiguous, the shape the indices broadcast to), the linear
// position in the indexed subspace (row-major over `sizes`) of every element goes to out, negative coordinates
// counting from the end (ref: misc.rs:150-203).
void index_positions(const hcb_tensor *out, int n, const hcb_tensor *const *coords, const int64_t *sizes, int32_t *bad_index,
                     int64_t *bad_value) {
    *bad_index = -1;
    *bad_value = 0;
    std::vector<std::vector<int64_t>> values;
    for (int k = 0; k < n; ++k) values.push_back(integers_of(*coords[k]));
    for (int k = 0; k < n; ++k) {
        for (int64_t v : values[static_cast<size_t>(k)]) {
            if (v < -sizes[k] || v >= sizes[k]) {
                *bad_index = k;
                *bad_value = v;
                return;
            }
        }
    }
    if (out == nullptr) return;
    const std::vector<int64_t> strides = contiguous_strides_of(sizes, n);
    // Every index, contiguous over its own shape, walked over out's shape (right-aligned, 1 -> stride 0).
    std::vector<std::vector<int64_t>> walks;
    for (int k = 0; k < n; ++k) {
        const hcb_tensor &c = *coords[k];
        const std::vector<int64_t> own = contiguous_strides_of(c.shape, c.ndim);
        std::vector<int64_t> walk(static_cast<size_t>(out->ndim), 0);
        for (int d = 0; d < c.ndim; ++d) {
            const int to = out->ndim - c.ndim + d;
            if (to < 0) panic("index_positions: an index has more dimensions than the positions");
            walk[static_cast<size_t>(to)] = c.shape[d] == 1 ? 0 : own[static_cast<size_t>(d)];
        }
        walks.push_back(walk);
    }
    int64_t *po = base<int64_t>(*out) + out->offset;
    const int64_t total = num_elements(*out);
    std::vector<int64_t> at(static_cast<size_t>(out->ndim), 0);
    for (int64_t e = 0; e < total; ++e) {
        int64_t position = 0;
        for (int k = 0; k < n; ++k) {
            int64_t offset = 0;
            for (int d = 0; d < out->ndim; ++d) offset += at[d] * walks[static_cast<size_t>(k)][static_cast<size_t>(d)];
            const int64_t v = values[static_cast<size_t>(k)][static_cast<size_t>(offset)];
            position += (v < 0 ? v + sizes[k] : v) * strides[static_cast<size_t>(k)];
        }
        po[e] = position;
        for (int d = out->ndim - 1; d >= 0; --d) {
            if (++at[d] < out->shape[d]) break;
            at[d] = 0;
        }
    }
}

template <class F>
int guarded(F f) {
    try {
        f();
        return 0;
    } catch (const Panic &p) {
        g_error = p.message;
        return 1;
    } catch (const std::exception &e) {
        g_error = std::string("internal error: ") + e.what();
        return 2;
    }
}

}  // namespace
}  // namespace orc

// ---- C entry points (loaded by the tests through ctypes, or plugged into the host layer) ------

extern "C" {

const char *orc_last_error(void) { return orc::g_error.c_str(); }

int orc_copy(const hcb_tensor *dst, const hcb_tensor *src) {
    return orc::guarded([&] { orc::copy(*dst, *src); });
}
int orc_fill(const hcb_tensor *dst, hcb_scalar value) {
    return orc::guarded([&] { orc::fill(*dst, value); });
}
int orc_unary(int32_t op, const hcb_tensor *out, const hcb_tensor *src) {
    return orc::guarded([&] { orc::unary(op, *out, *src); });
}
int orc_binary(int32_t op, const hcb_tensor *out, const hcb_tensor *a, const hcb_tensor *b) {
    return orc::guarded([&] { orc::binary(op, *out, *a, *b); });
}
int orc_binary_constant(int32_t op, const hcb_tensor *out, const hcb_tensor *a, hcb_scalar value,
                        int32_t constant_first) {
    return orc::guarded([&] { orc::binary_constant(op, *out, *a, value, constant_first != 0); });
}
int orc_binary_scalar(int32_t op, const hcb_tensor *out, const hcb_tensor *a, double s, int32_t scalar_first) {
    return orc::guarded([&] { orc::binary_scalar(op, *out, *a, s, scalar_first != 0); });
}
int orc_where(const hcb_tensor *out, const hcb_tensor *cond, const hcb_tensor *x, const hcb_tensor *y) {
    return orc::guarded([&] { orc::where_(*out, *cond, *x, *y); });
}
int orc_where_constant(const hcb_tensor *out, const hcb_tensor *cond, const hcb_tensor *x, hcb_scalar xv,
                       const hcb_tensor *y, hcb_scalar yv) {
    return orc::guarded([&] { orc::where_constant(*out, *cond, x, xv, y, yv); });
}
int orc_reduce(int32_t op, const hcb_tensor *out, const hcb_tensor *src, const uint8_t *mask) {
    return orc::guarded([&] { orc::reduce(op, *out, *src, mask); });
}
int orc_var(const hcb_tensor *out, const hcb_tensor *src, const uint8_t *mask, double correction,
            int32_t take_sqrt) {
    return orc::guarded([&] { orc::var(*out, *src, mask, correction, take_sqrt != 0); });
}
int orc_arg_reduce(const hcb_tensor *values, const hcb_tensor *indices, const hcb_tensor *src, int32_t dim,
                   int32_t is_max) {
    return orc::guarded([&] { orc::arg_reduce(values, *indices, *src, dim, is_max != 0); });
}
int orc_softmax(const hcb_tensor *out, const hcb_tensor *src, int32_t dim, int32_t log) {
    return orc::guarded([&] { orc::softmax(*out, *src, dim, log != 0); });
}

int orc_fused(int32_t kind, double scalar, const hcb_tensor *out, const hcb_tensor *a, const hcb_tensor *b,
              const hcb_tensor *c) {
    return orc::guarded([&] { orc::fused(kind, scalar, *out, *a, *b, c); });
}
int orc_triangle(const hcb_tensor *out, const hcb_tensor *src, int64_t diagonal, int32_t upper) {
    return orc::guarded([&] { orc::triangle(*out, *src, diagonal, upper != 0); });
}
int orc_flip(const hcb_tensor *out, const hcb_tensor *src, const uint8_t *mask) {
    return orc::guarded([&] { orc::flip(*out, *src, mask); });
}
int orc_exclusive_cumprod(const hcb_tensor *out, const hcb_tensor *src, int32_t dim, int32_t reverse) {
    return orc::guarded([&] { orc::exclusive_cumprod(*out, *src, dim, reverse != 0); });
}
void orc_philox(const uint32_t *counter, const uint32_t *key, uint32_t *out) { orc::philox(counter, key, out); }
int orc_random_uniform(const hcb_tensor *out, uint64_t seed, uint64_t offset, double from, double to) {
    return orc::guarded([&] { orc::random_uniform(*out, seed, offset, from, to); });
}
int orc_random_normal(const hcb_tensor *out, uint64_t seed, uint64_t offset, double mean, double std) {
    return orc::guarded([&] { orc::random_normal(*out, seed, offset, mean, std); });
}
int orc_random_int(const hcb_tensor *out, uint64_t seed, uint64_t offset, uint64_t blocks, int64_t low, uint64_t range,
                   uint64_t threshold, uint64_t *accepted) {
    return orc::guarded([&] { *accepted = orc::random_int(*out, seed, offset, blocks, low, range, threshold); });
}
int orc_index_select(const hcb_tensor *out, const hcb_tensor *src, int32_t dim, const hcb_tensor *index, int32_t bounds) {
    return orc::guarded([&] { orc::index_select(*out, *src, dim, *index, bounds); });
}
int orc_gather(const hcb_tensor *out, const hcb_tensor *src, int32_t dim, const hcb_tensor *index) {
    return orc::guarded([&] { orc::gather(*out, *src, dim, *index); });
}
int orc_index_add(const hcb_tensor *out, int32_t dim, const hcb_tensor *index, const hcb_tensor *src, int32_t bounds) {
    return orc::guarded([&] { orc::index_add(*out, dim, *index, *src, bounds); });
}
int orc_scatter_add(const hcb_tensor *out, int32_t dim, const hcb_tensor *index, const hcb_tensor *src) {
    return orc::guarded([&] { orc::scatter_add(*out, dim, *index, *src); });
}
int orc_index_overwrite(const hcb_tensor *out, int32_t dim, const hcb_tensor *index, const hcb_tensor *src) {
    return orc::guarded([&] { orc::index_overwrite(*out, dim, *index, *src); });
}
int orc_mask_coordinates(const hcb_tensor *mask, const hcb_tensor *out, int64_t *count) {
    return orc::guarded([&] { *count = orc::mask_coordinates(*mask, out); });
}
int orc_index_positions(const hcb_tensor *out, int32_t n, const hcb_tensor *const *coords, const int64_t *sizes, int32_t *bad_index,
                        int64_t *bad_value) {
    return orc::guarded([&] { orc::index_positions(out, n, coords, sizes, bad_index, bad_value); });
}
int orc_addr(const hcb_tensor *out, const hcb_tensor *v1, const hcb_tensor *v2, const hcb_tensor *input, hcb_scalar alpha,
             hcb_scalar beta) {
    return orc::guarded([&] { orc::addr(*out, *v1, *v2, *input, alpha, beta); });
}

// erf in f64, for the known-answer table of ref: src/backend/cpu/num.rs:225-248.
double orc_erf(double x) { return orc::erf64(x); }

// Integer power, for ref: src/backend/cpu/num.rs:250-257.
int64_t orc_int_pow_i64(int64_t b, int64_t e) { return orc::int_pow<int64_t>(b, e); }
int32_t orc_int_pow_i32(int32_t b, int32_t e) { return orc::int_pow<int32_t>(b, e); }
int8_t orc_int_pow_i8(int8_t b, int8_t e) { return orc::int_pow<int8_t>(b, e); }

// The table a process hands to the host layer to run kernels on CPU tensors.
const hcb_backend *orc_backend(void) {
    static const hcb_backend table = {
        "homura CPU oracle", orc_last_error, orc_copy,  orc_fill,           orc_unary,
        orc_binary,          orc_binary_constant,       orc_binary_scalar,  orc_where,
        orc_where_constant,  orc_reduce,     orc_var,   orc_arg_reduce,     orc_softmax,
        orc_fused,           orc_triangle,   orc_flip,  orc_addr,           orc_exclusive_cumprod,
        orc_random_uniform,  orc_random_normal,         orc_random_int,
        orc_index_select,    orc_gather,     orc_index_add,         orc_scatter_add,
        orc_index_overwrite, orc_mask_coordinates,      orc_index_positions,
    };
    return &table;
}

}  // extern "C"
