// The integer kernels of hmr_binary / hmr_binary_constant (see ew_binary.hip).
#include "ew_common.hpp"

namespace hmr {

bool launch_int_binary(int op, int dtype, const MapCall &call, hipStream_t stream) {
    using IntOps = std::integer_sequence<int, HMR_BINARY_ADD, HMR_BINARY_SUB, HMR_BINARY_MUL, HMR_BINARY_POW,
                                         HMR_BINARY_MAXIMUM, HMR_BINARY_MINIMUM, HMR_BINARY_BITWISE_AND>;
    bool done = false;
    with_int_type(dtype, [&](auto t) {
        using T = typename decltype(t)::type;
        done = with_code(op, IntOps{}, [&](auto o) { launch_map<IntBinary<decltype(o)::value, T>>(call, stream); });
    });
    return done;
}

}  // namespace hmr
