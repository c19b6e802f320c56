// Integer / bool sum and product (into I64, wrapping) and the truth folds all / any.
#include "dispatch.hpp"
#include "reduce_plan.hpp"

namespace hmr {

bool launch_int_reduce(int op, int dtype, const ReducePlan &plan, void *partials, void *out, hipStream_t stream) {
    if (dtype >= HMR_F16) return false;
    return with_any_type(dtype, [&](auto t) {
        using T = typename decltype(t)::type;
        if constexpr (Conv<T>::kind != Kind::Float) {
            I64Sink sink{static_cast<int64_t *>(out)};
            if (op == HMR_REDUCE_PROD) launch_reduce(plan, partials, IntFold<T, true>{}, sink, stream);
            else launch_reduce(plan, partials, IntFold<T, false>{}, sink, stream);
        }
    });
}

bool launch_truth_reduce(int op, int dtype, const ReducePlan &plan, void *partials, void *out, hipStream_t stream) {
    return with_any_type(dtype, [&](auto t) {
        using T = typename decltype(t)::type;
        TruthSink sink{static_cast<uint8_t *>(out)};
        if (op == HMR_REDUCE_ALL) launch_reduce(plan, partials, TruthFold<T, true>{}, sink, stream);
        else launch_reduce(plan, partials, TruthFold<T, false>{}, sink, stream);
    });
}

}  // namespace hmr
