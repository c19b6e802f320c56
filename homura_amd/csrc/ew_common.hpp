// Glue between the C entry points and launch_map: checks, early exits, launch bracket.
#pragma once

#include "dispatch.hpp"
#include "map.hpp"
#include "ops.hpp"

namespace hmr {

// Runs an elementwise entry point: prepares the call from `descs` (nullptr = constant), returns
// early for empty tensors, and launches through `pick`, which returns false when there is no
// kernel for the dtypes/op.
// `before(call)` runs after the checks and before the launch bracket; it may fail the call.
template <class Pick, class Before>
hmr_status run_map(hmr_context_t ctx, const char *what, int count, const hmr_tensor_desc *const *descs,
                   const uint64_t *bits, Pick pick, Before before, bool negative_inputs = false) {
    MapCall call;
    if (hmr_status s = prepare_map(call, count, descs, bits, negative_inputs)) return s;
    if (call.n == 0) return HMR_OK;
    if (ctx == nullptr) return fail(HMR_INVALID, std::string(what) + ": null context");
    call.compute_units = ctx->compute_units;
    if (hmr_status s = before(call)) return s;
    return queue_on(ctx, what, [&](hipStream_t stream) { return pick(call, stream); });
}

template <class Pick>
hmr_status run_map(hmr_context_t ctx, const char *what, int count, const hmr_tensor_desc *const *descs,
                   const uint64_t *bits, Pick pick) {
    return run_map(ctx, what, count, descs, bits, pick, [](const MapCall &) { return HMR_OK; });
}

// The same-dtype arithmetic kernels of hmr_binary, one translation unit per family (ew_binary_int.hip,
// ew_binary_float.hip); false when there is no kernel for the op and dtype.
bool launch_int_binary(int op, int dtype, const MapCall &call, hipStream_t stream);
bool launch_float_binary(int op, int dtype, const MapCall &call, hipStream_t stream);

}  // namespace hmr
