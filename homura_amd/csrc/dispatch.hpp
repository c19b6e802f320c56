// Run-time value -> compile-time tag selection for dtypes and op codes.
#pragma once

#include <utility>

#include "elem.hpp"

namespace hmr {

template <class T>
struct TypeTag {
    using type = T;
};

template <int V>
struct IntTag {
    static constexpr int value = V;
};

// Calls f(TypeTag<T>{}) for the storage type of `dtype` when it is in the family; returns false
// (calling nothing) otherwise.
template <class F>
bool with_float_type(int dtype, F &&f) {
    switch (dtype) {
        case HMR_F16: f(TypeTag<f16_t>{}); return true;
        case HMR_BF16: f(TypeTag<bf16_t>{}); return true;
        case HMR_F32: f(TypeTag<float>{}); return true;
        case HMR_F64: f(TypeTag<double>{}); return true;
        default: return false;
    }
}

template <class F>
bool with_int_type(int dtype, F &&f) {
    switch (dtype) {
        case HMR_U8: f(TypeTag<uint8_t>{}); return true;
        case HMR_I8: f(TypeTag<int8_t>{}); return true;
        case HMR_I16: f(TypeTag<int16_t>{}); return true;
        case HMR_I32: f(TypeTag<int32_t>{}); return true;
        case HMR_I64: f(TypeTag<int64_t>{}); return true;
        default: return false;
    }
}

template <class F>
bool with_any_type(int dtype, F &&f) {
    if (dtype == HMR_BOOL) {
        f(TypeTag<bool_t>{});
        return true;
    }
    return with_int_type(dtype, f) || with_float_type(dtype, f);
}

// Unsigned word of an element size, for ops that only move bits.
template <class F>
bool with_word(int size, F &&f) {
    switch (size) {
        case 1: f(TypeTag<uint8_t>{}); return true;
        case 2: f(TypeTag<uint16_t>{}); return true;
        case 4: f(TypeTag<uint32_t>{}); return true;
        case 8: f(TypeTag<uint64_t>{}); return true;
        default: return false;
    }
}

// Calls f(IntTag<V>{}) for the V among Vs equal to `value`.
template <int... Vs, class F>
bool with_code(int value, std::integer_sequence<int, Vs...>, F &&f) {
    return ((value == Vs ? (f(IntTag<Vs>{}), true) : false) || ...);
}

}  // namespace hmr
