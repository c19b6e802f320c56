// max / min with the value and, for the arg reductions, the position of the winner.
#include "dispatch.hpp"
#include "reduce_plan.hpp"

namespace hmr {

bool launch_extreme_reduce(bool is_max, int dtype, const ReducePlan &plan, void *partials, void *values,
                           void *indices, hipStream_t stream) {
    return with_any_type(dtype, [&](auto t) {
        using T = typename decltype(t)::type;
        ExtremeSink<T> sink{static_cast<T *>(values), static_cast<int64_t *>(indices)};
        if (is_max) launch_reduce(plan, partials, ExtremeFold<T, true>{}, sink, stream);
        else launch_reduce(plan, partials, ExtremeFold<T, false>{}, sink, stream);
    });
}

}  // namespace hmr
