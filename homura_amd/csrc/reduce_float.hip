// Float sum / product / mean and the two variance passes, for the four float dtypes.
#include "dispatch.hpp"
#include "reduce_plan.hpp"

namespace hmr {

bool launch_float_reduce(int op, int dtype, const ReducePlan &plan, void *partials, void *out, hipStream_t stream) {
    return with_float_type(dtype, [&](auto t) {
        using T = typename decltype(t)::type;
        T *o = static_cast<T *>(out);
        if (op == HMR_REDUCE_PROD) {
            launch_reduce(plan, partials, FloatFold<T, true>{}, RoundSink<T, false>{o}, stream);
        } else if (op == HMR_REDUCE_SUM) {
            launch_reduce(plan, partials, FloatFold<T, false>{}, RoundSink<T, false>{o}, stream);
        } else {
            launch_reduce(plan, partials, FloatFold<T, false>{}, RoundSink<T, true>{o}, stream);
        }
    });
}

bool launch_mean_pass(int dtype, const ReducePlan &plan, void *partials, double *means, hipStream_t stream) {
    return with_float_type(dtype, [&](auto t) {
        using T = typename decltype(t)::type;
        launch_reduce(plan, partials, FloatFold<T, false>{}, MeanSink{means}, stream);
    });
}

bool launch_deviation_pass(int dtype, const ReducePlan &plan, void *partials, const double *means, void *out,
                           double divisor, bool take_sqrt, hipStream_t stream) {
    return with_float_type(dtype, [&](auto t) {
        using T = typename decltype(t)::type;
        launch_reduce(plan, partials, DeviationFold<T>{means}, VarSink<T>{static_cast<T *>(out), divisor, take_sqrt},
                      stream);
    });
}

}  // namespace hmr
