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

// Rows plan, one slice, and a row that fits G lanes x 16 tiles of 16 bytes: registers.
static int var_row_tiles(const ReducePlan &plan, int elem) {
    if (plan.kind != ReduceKind::Rows || plan.splits != 1 || plan.args.runs.dims != 0) return 0;
    const int64_t vec = 16 / elem;
    if (plan.args.nred % vec != 0) return 0;  // the register kernel takes whole 16-byte chunks
    const int64_t per = (plan.args.nred + vec * plan.group - 1) / (vec * plan.group);
    return per <= 4 ? 4 : (per <= 8 ? 8 : (per <= 16 ? 16 : 0));
}

bool launch_var_single_pass(int dtype, const ReducePlan &plan, void *partials, void *out, double divisor,
                            bool take_sqrt, hipStream_t stream) {
    if (plan.args.nred == 0) return false;
    bool done = false;
    with_float_type(dtype, [&](auto t) {
        using T = typename decltype(t)::type;
        VarSink<T> sink{static_cast<T *>(out), divisor, take_sqrt};
        if (plan.kind == ReduceKind::Cols) {
            // The shifted one-pass sums lose about a factor n when a column's first element lies far from its
            // mean. In f64 arithmetic that is nothing next to an ulp of an f16, bf16 or f32 result; an f64
            // result is held to 4 n eps of the variance itself, so f64 columns take the two passes.
            if constexpr (std::is_same_v<T, double>) return;
            launch_reduce(plan, partials, MomentsFold<T>{}, sink, stream);
            done = true;
            return;
        }
        const int tiles = var_row_tiles(plan, static_cast<int>(sizeof(T)));
        if (tiles == 0) {
            // Rows that do not fit the registers - made of several runs, or cut into slices -: the same one pass
            // of shifted sums (every lane about its own first element, merged by Chan's formula) instead of two
            // passes over memory; f64 results keep the two passes, as for columns.
            if (plan.kind == ReduceKind::Rows && (plan.args.runs.dims != 0 || plan.splits > 1) && !std::is_same_v<T, double>) {
                launch_reduce(plan, partials, MomentsFold<T>{}, sink, stream);
                done = true;
            }
            return;
        }
        ReduceArgs a = plan.args;
        a.splits = 1;
        a.chunk = a.nred;
        const int64_t cap = 1 << 20;
        auto run = [&](auto w, auto c) {
            constexpr int W = decltype(w)::value, C = decltype(c)::value;
            dim3 grid(capped((a.nout + (4 / W) - 1) / (4 / W), cap));
            hipLaunchKernelGGL((var_rows_kernel<T, W, C>), grid, dim3(kBlock), 0, stream, a, sink);
        };
        auto with_tiles = [&](auto w) {
            if (tiles == 4) run(w, IntTag<4>{});
            else if (tiles == 8) run(w, IntTag<8>{});
            else run(w, IntTag<16>{});
        };
        if (plan.group == kWave) with_tiles(IntTag<1>{});
        else with_tiles(IntTag<4>{});
        done = true;
    });
    return done;
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
