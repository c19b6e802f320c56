// Host-side planning of a reduction and the typed launch of its kernels.
#pragma once

#include "dispatch.hpp"
#include "reduce.hpp"

namespace hmr {

enum class ReduceKind { Any, Rows, Cols };

// How a reduction runs. Depends only on sizes, strides, the element size and alignment, never on
// values or timing (ref: csrc/reduce.hpp:12-14 gives the same guarantee for the reference's plans).
struct ReducePlan {
    ReduceKind kind = ReduceKind::Any;
    int group = 1;        // lanes per output: 1, 64 or 256 (Cols: 4 waves share 64*V outputs -> reported as 4)
    int64_t splits = 1;   // slices of the reduced range
    int64_t chunk = 0;    // reduced elements per slice
    int64_t rstride = 0;  // Cols: stride of the reduced dimension
    int64_t inner = 0;    // Cols: length of the contiguous run of outputs
    int across = 4;       // Cols: waves side by side on a column span (1, 2 or 4)
    ReduceArgs args{};    // src, walks, counts (partials filled in at launch)
};

// Bytes one partial accumulator occupies in the workspace, whatever the op: a value + position
// pair at most, or for hmr_var a (count, mean, M2) triple.
constexpr int64_t kPartialBytes = 16;
constexpr int64_t kVarPartialBytes = 32;
// Machine width the plans aim at: lanes of a full MI355X at 4 waves per SIMD.
constexpr int64_t kTargetLanes = 256 * 4 * 4 * 64;

// Checks the descriptions of a reduction (ref: csrc/reduce.hip:133-160) and plans it. `out` may
// be null (size queries); otherwise it must be contiguous over kept's sizes.
hmr_status plan_reduction(const hmr_tensor_desc *out, const hmr_tensor_desc &kept, const hmr_tensor_desc &red,
                          ReducePlan &plan);

// Workspace: [f64 means for hmr_var when nout > 0][partials when splits > 1].
int64_t means_bytes(const ReducePlan &p, bool var);
int64_t partial_bytes(const ReducePlan &p, bool var);

inline unsigned capped(int64_t blocks, int64_t cap) {
    if (blocks < 1) blocks = 1;
    return static_cast<unsigned>(blocks < cap ? blocks : cap);
}

// Launches the planned kernels for one (op, sink) pair on `stream`.
template <class Op, class Sink>
void launch_reduce(const ReducePlan &plan, void *partials, Op op, Sink sink, hipStream_t stream) {
    using Acc = typename Op::Acc;
    static_assert(sizeof(Acc) <= (std::is_same_v<Acc, Moments> ? kVarPartialBytes : kPartialBytes), "partial slot too small");
    ReduceArgs a = plan.args;
    a.splits = plan.splits;
    a.chunk = plan.chunk;
    a.partials = partials;
    const int64_t cap = 1 << 20;
    const unsigned ysplits = static_cast<unsigned>(plan.splits);
    switch (plan.kind) {
        case ReduceKind::Rows: {
            if (plan.group == kWave) {
                dim3 grid(capped((a.nout + 3) / 4, cap), ysplits);
                hipLaunchKernelGGL((reduce_rows_kernel<Op, Sink, 1>), grid, dim3(kBlock), 0, stream, a, op, sink);
            } else {
                dim3 grid(capped(a.nout, cap), ysplits);
                hipLaunchKernelGGL((reduce_rows_kernel<Op, Sink, 4>), grid, dim3(kBlock), 0, stream, a, op, sink);
            }
            break;
        }
        case ReduceKind::Cols: {
            constexpr int V = 16 / static_cast<int>(sizeof(typename Op::In));
            int64_t span = int64_t{plan.across} * kWave * V;
            int64_t tiles = (plan.inner + span - 1) / span * (a.nout / plan.inner);
            dim3 grid(capped(tiles, cap), ysplits);
            if (plan.group == 1024 / kWave) {
                // Planned for elements of four bytes or more (the states of wider tiles would not fit LDS).
                if constexpr (sizeof(typename Op::In) >= 4) {
                    hipLaunchKernelGGL((reduce_cols_kernel<Op, Sink, 1024>), grid, dim3(1024), 0, stream, a,
                                       plan.rstride, plan.inner, plan.across, op, sink);
                }
            } else {
                hipLaunchKernelGGL((reduce_cols_kernel<Op, Sink, kBlock>), grid, dim3(kBlock), 0, stream, a,
                                   plan.rstride, plan.inner, plan.across, op, sink);
            }
            break;
        }
        case ReduceKind::Any: {
            if (plan.group == 1) {
                dim3 grid(capped((a.nout + kBlock - 1) / kBlock, cap), ysplits);
                hipLaunchKernelGGL((reduce_any_kernel<Op, Sink, 1>), grid, dim3(kBlock), 0, stream, a, op, sink);
            } else if (plan.group == kWave) {
                dim3 grid(capped((a.nout + 3) / 4, cap), ysplits);
                hipLaunchKernelGGL((reduce_any_kernel<Op, Sink, kWave>), grid, dim3(kBlock), 0, stream, a, op, sink);
            } else {
                dim3 grid(capped(a.nout, cap), ysplits);
                hipLaunchKernelGGL((reduce_any_kernel<Op, Sink, kBlock>), grid, dim3(kBlock), 0, stream, a, op, sink);
            }
            break;
        }
    }
    if (plan.splits > 1) {
        // Outputs per workgroup: as many as still leave a workgroup per compute unit.
        auto run = [&](auto outs) {
            constexpr int OUTS = decltype(outs)::value;
            hipLaunchKernelGGL((combine_kernel<Op, Sink, OUTS>), dim3(capped((a.nout + OUTS - 1) / OUTS, cap)),
                               dim3(kBlock), 0, stream, a, op, sink);
        };
        if (a.nout >= 64 * 256) run(IntTag<64>{});
        else if (a.nout >= 16 * 256) run(IntTag<16>{});
        else if (a.nout >= 4 * 64) run(IntTag<4>{});
        else run(IntTag<1>{});
    }
}

// Typed launchers, one translation unit per accumulator family. Each returns false when it has
// no kernel for the dtype/op pair (and then queues nothing).
bool launch_float_reduce(int op, int dtype, const ReducePlan &plan, void *partials, void *out, hipStream_t stream);
bool launch_int_reduce(int op, int dtype, const ReducePlan &plan, void *partials, void *out, hipStream_t stream);
bool launch_truth_reduce(int op, int dtype, const ReducePlan &plan, void *partials, void *out, hipStream_t stream);
bool launch_extreme_reduce(bool is_max, int dtype, const ReducePlan &plan, void *partials, void *values,
                           void *indices, hipStream_t stream);
// Variance in one launch where the plan allows it (rows that fit in registers; columns in one
// pass over memory); false when the two-pass form below has to run.
bool launch_var_single_pass(int dtype, const ReducePlan &plan, void *partials, void *out, double divisor,
                            bool take_sqrt, hipStream_t stream);
// The two passes of the variance: means (f64) then squared deviations.
bool launch_mean_pass(int dtype, const ReducePlan &plan, void *partials, double *means, hipStream_t stream);
bool launch_deviation_pass(int dtype, const ReducePlan &plan, void *partials, const double *means, void *out,
                           double divisor, bool take_sqrt, hipStream_t stream);

}  // namespace hmr
