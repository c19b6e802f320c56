// hmr_binary_scalar, hmr_where, hmr_where_constant, hmr_fill
// (ref: csrc/homura_rocm.h:142, 217, 247-255; csrc/elementwise.hip:1035-1132, csrc/copy.hip:154-173).
#include "ew_common.hpp"

namespace hmr {
namespace {

template <class T>
uint64_t scalar_bits_of(double s) {
    using C = typename Comp<T>::C;
    C c = static_cast<C>(s);  // rounded to the computation type, as the CPU's C::of
    uint64_t bits = 0;
    __builtin_memcpy(&bits, &c, sizeof c);
    return bits;
}

}  // namespace
}  // namespace hmr

extern "C" {

hmr_status hmr_binary_scalar(hmr_context_t ctx, int32_t op, const hmr_tensor_desc *out, const hmr_tensor_desc *a,
                             double s, int32_t scalar_first) {
    return hmr::guarded([&] {
        if (op != HMR_BINARY_MUL && op != HMR_BINARY_DIV) {
            return hmr::fail(HMR_INVALID, "binary_scalar: only Mul and Div keep their scalar unrounded");
        }
        const int mode = op == HMR_BINARY_MUL ? 0 : (scalar_first ? 2 : 1);
        uint64_t bits = 0;
        bool is_float = hmr::with_float_type(a->dtype, [&](auto t) {
            bits = hmr::scalar_bits_of<typename decltype(t)::type>(s);
        });
        const hmr_tensor_desc *descs[3] = {out, a, nullptr};
        const uint64_t cbits[3] = {0, 0, bits};
        return hmr::run_map(ctx, "binary_scalar", 3, descs, cbits,
                            [&](const hmr::MapCall &call, hipStream_t stream) {
                                if (!is_float || out->dtype != a->dtype) return false;
                                return hmr::with_float_type(a->dtype, [&](auto t) {
                                    using T = typename decltype(t)::type;
                                    if (mode == 0) hmr::launch_map<hmr::ScalarBinary<0, T>>(call, stream);
                                    else if (mode == 1) hmr::launch_map<hmr::ScalarBinary<1, T>>(call, stream);
                                    else hmr::launch_map<hmr::ScalarBinary<2, T>>(call, stream);
                                });
                            });
    });
}

hmr_status hmr_where_constant(hmr_context_t ctx, const hmr_tensor_desc *out, const hmr_tensor_desc *cond,
                              const hmr_tensor_desc *x, uint64_t x_bits, const hmr_tensor_desc *y,
                              uint64_t y_bits) {
    return hmr::guarded([&] {
        const hmr_tensor_desc *descs[4] = {out, cond, x, y};
        const uint64_t cbits[4] = {0, 0, x_bits, y_bits};
        return hmr::run_map(ctx, "where", 4, descs, cbits, [&](const hmr::MapCall &call, hipStream_t stream) {
            if (cond->dtype != HMR_BOOL) return false;
            if ((x && x->dtype != out->dtype) || (y && y->dtype != out->dtype)) return false;
            return hmr::with_word(hmr::dtype_size(out->dtype), [&](auto w) {
                hmr::launch_map<hmr::Select<typename decltype(w)::type>>(call, stream);
            });
        });
    });
}

hmr_status hmr_where(hmr_context_t ctx, const hmr_tensor_desc *out, const hmr_tensor_desc *cond,
                     const hmr_tensor_desc *x, const hmr_tensor_desc *y) {
    if (x == nullptr || y == nullptr) return hmr::fail(HMR_INVALID, "where: a branch is missing");
    return hmr_where_constant(ctx, out, cond, x, 0, y, 0);
}

hmr_status hmr_fill(hmr_context_t ctx, const hmr_tensor_desc *dst, uint64_t bits) {
    return hmr::guarded([&] {
        const hmr_tensor_desc *descs[2] = {dst, nullptr};
        const uint64_t cbits[2] = {0, bits};
        return hmr::run_map(ctx, "fill", 2, descs, cbits, [&](const hmr::MapCall &call, hipStream_t stream) {
            return hmr::with_word(hmr::dtype_size(dst->dtype), [&](auto w) {
                hmr::launch_map<hmr::Move<typename decltype(w)::type>>(call, stream);
            });
        });
    });
}

}  // extern "C"
