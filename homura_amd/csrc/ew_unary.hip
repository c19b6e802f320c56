// hmr_unary (ref: csrc/homura_rocm.h:202, csrc/elementwise.hip:996-1007).
#include "ew_common.hpp"

namespace hmr {
namespace {

using FloatOps = std::integer_sequence<int, HMR_UNARY_NEG, HMR_UNARY_ABS, HMR_UNARY_SIGN, HMR_UNARY_RELU,
                                       HMR_UNARY_EXP, HMR_UNARY_LOG, HMR_UNARY_SQRT, HMR_UNARY_RSQRT,
                                       HMR_UNARY_RECIPROCAL, HMR_UNARY_SIN, HMR_UNARY_COS, HMR_UNARY_ERF,
                                       HMR_UNARY_TANH, HMR_UNARY_SIGMOID, HMR_UNARY_LOG_SIGMOID, HMR_UNARY_SILU,
                                       HMR_UNARY_GELU, HMR_UNARY_GELU_TANH>;
using IntOps = std::integer_sequence<int, HMR_UNARY_NEG, HMR_UNARY_ABS, HMR_UNARY_SIGN, HMR_UNARY_RELU>;

bool pick_unary(int op, int out_dtype, int dtype, const MapCall &call, hipStream_t stream) {
    if (op == HMR_UNARY_LOGICAL_NOT) {
        if (out_dtype != HMR_BOOL) return false;
        return with_any_type(dtype, [&](auto t) {
            using T = typename decltype(t)::type;
            launch_map<LogicalNot<T>>(call, stream);
        });
    }
    if (out_dtype != dtype) return false;
    if (dtype == HMR_BOOL) {
        if (op != HMR_UNARY_SIGN) return false;  // the CPU has no other bool arm
        launch_map<Move<uint8_t>>(call, stream);
        return true;
    }
    bool done = false;
    if (with_int_type(dtype, [&](auto t) {
            using T = typename decltype(t)::type;
            done = with_code(op, IntOps{}, [&](auto o) { launch_map<UnaryInt<decltype(o)::value, T>>(call, stream); });
        })) {
        return done;
    }
    with_float_type(dtype, [&](auto t) {
        using T = typename decltype(t)::type;
        done = with_code(op, FloatOps{}, [&](auto o) { launch_map<UnaryFloat<decltype(o)::value, T>>(call, stream); });
    });
    return done;
}

}  // namespace
}  // namespace hmr

extern "C" hmr_status hmr_unary(hmr_context_t ctx, int32_t op, const hmr_tensor_desc *out,
                                const hmr_tensor_desc *src) {
    return hmr::guarded([&] {
        const hmr_tensor_desc *descs[2] = {out, src};
        return hmr::run_map(ctx, "unary", 2, descs, nullptr, [&](const hmr::MapCall &call, hipStream_t stream) {
            return hmr::pick_unary(op, out->dtype, src->dtype, call, stream);
        });
    });
}
