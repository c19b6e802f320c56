// hmr_binary and hmr_binary_constant (ref: csrc/homura_rocm.h:206-213,
// csrc/elementwise.hip:1009-1033). A constant operand travels as a kernel argument.
#include "ew_common.hpp"

namespace hmr {
namespace {

using CompareOps = std::integer_sequence<int, HMR_BINARY_GREATER, HMR_BINARY_GREATER_EQUAL, HMR_BINARY_LESS,
                                         HMR_BINARY_LESS_EQUAL, HMR_BINARY_EQUAL, HMR_BINARY_NOT_EQUAL>;
using MixedOps = std::integer_sequence<int, HMR_BINARY_ADD, HMR_BINARY_SUB, HMR_BINARY_MUL, HMR_BINARY_DIV>;

// Mixed float inputs (extension): a half with F32, output F32.
template <class A, class B>
bool pick_mixed(int op, const MapCall &call, hipStream_t stream) {
    return with_code(op, MixedOps{},
                     [&](auto o) { launch_map<FloatBinary<decltype(o)::value, float, A, B>>(call, stream); });
}

bool pick_binary(int op, int out_dtype, int a_dtype, int b_dtype, const MapCall &call, hipStream_t stream) {
    if (a_dtype != b_dtype) {
        if (out_dtype != HMR_F32) return false;
        if (a_dtype == HMR_BF16 && b_dtype == HMR_F32) return pick_mixed<bf16_t, float>(op, call, stream);
        if (a_dtype == HMR_F32 && b_dtype == HMR_BF16) return pick_mixed<float, bf16_t>(op, call, stream);
        if (a_dtype == HMR_F16 && b_dtype == HMR_F32) return pick_mixed<f16_t, float>(op, call, stream);
        if (a_dtype == HMR_F32 && b_dtype == HMR_F16) return pick_mixed<float, f16_t>(op, call, stream);
        return false;
    }
    const int dtype = a_dtype;
    bool done = false;
    if (op >= HMR_BINARY_GREATER && op <= HMR_BINARY_NOT_EQUAL) {
        if (out_dtype != HMR_BOOL) return false;
        with_any_type(dtype, [&](auto t) {
            using T = typename decltype(t)::type;
            done = with_code(op, CompareOps{}, [&](auto o) { launch_map<Compare<decltype(o)::value, T>>(call, stream); });
        });
        return done;
    }
    if (op == HMR_BINARY_LOGICAL_AND || op == HMR_BINARY_LOGICAL_OR) {
        if (out_dtype != HMR_BOOL || dtype != HMR_BOOL) return false;
        if (op == HMR_BINARY_LOGICAL_AND) launch_map<BoolBinary<true>>(call, stream);
        else launch_map<BoolBinary<false>>(call, stream);
        return true;
    }
    if (out_dtype != dtype) return false;
    if (dtype == HMR_BOOL) {
        switch (op) {
            case HMR_BINARY_ADD:
            case HMR_BINARY_MAXIMUM: launch_map<BoolBinary<false>>(call, stream); return true;
            case HMR_BINARY_MUL:
            case HMR_BINARY_MINIMUM:
            case HMR_BINARY_BITWISE_AND: launch_map<BoolBinary<true>>(call, stream); return true;
            default: return false;
        }
    }
    // Same-dtype arithmetic: the integer and the float kernels are translation units of their own.
    if (dtype >= HMR_U8 && dtype <= HMR_I64) return launch_int_binary(op, dtype, call, stream);
    return launch_float_binary(op, dtype, call, stream);
}

}  // namespace
}  // namespace hmr

extern "C" {

hmr_status hmr_binary(hmr_context_t ctx, int32_t op, const hmr_tensor_desc *out, const hmr_tensor_desc *a,
                      const hmr_tensor_desc *b) {
    return hmr::fenced([&] {
        const hmr_tensor_desc *descs[3] = {out, a, b};
        return hmr::run_map(ctx, "binary", 3, descs, nullptr, [&](const hmr::MapCall &call, hipStream_t stream) {
            return hmr::pick_binary(op, out->dtype, a->dtype, b->dtype, call, stream);
        });
    });
}

hmr_status hmr_binary_constant(hmr_context_t ctx, int32_t op, const hmr_tensor_desc *out, const hmr_tensor_desc *a,
                               uint64_t bits, int32_t constant_first) {
    return hmr::fenced([&] {
        const hmr_tensor_desc *descs[3] = {out, constant_first ? nullptr : a, constant_first ? a : nullptr};
        const uint64_t cbits[3] = {0, bits, bits};
        return hmr::run_map(ctx, "binary_constant", 3, descs, cbits,
                            [&](const hmr::MapCall &call, hipStream_t stream) {
                                return hmr::pick_binary(op, out->dtype, a->dtype, a->dtype, call, stream);
                            });
    });
}

}  // extern "C"
