// Entry points of kernel families this library does not implement (see homura_rocm_unbuilt.h).
// Exported so that every `extern "C"` declaration of the reference's Rust bindings resolves;
// each fails with HMR_INVALID and queues nothing.
#include "common.hpp"
#include "homura_rocm_unbuilt.h"

namespace {
hmr_status unbuilt(const char *name) {
    return hmr::fenced([&] { return hmr::fail(HMR_INVALID, std::string(name) + ": not built in this library"); });
}
}  // namespace

#define HMR_UNBUILT(NAME, ...) \
    hmr_status NAME(__VA_ARGS__) { return unbuilt(#NAME); }

extern "C" {

HMR_UNBUILT(hmr_max_pool2d_backward_workspace, int64_t, int64_t *)
HMR_UNBUILT(hmr_max_pool2d_backward, hmr_context_t, const hmr_tensor_desc *, const hmr_tensor_desc *,
            const hmr_tensor_desc *, void *, int64_t)
HMR_UNBUILT(hmr_max_pool2d, hmr_context_t, const hmr_tensor_desc *, const hmr_tensor_desc *,
            const hmr_tensor_desc *, const int64_t *)
HMR_UNBUILT(hmr_max_pool2d_check, hmr_context_t, const hmr_tensor_desc *, int64_t, int64_t, const int64_t *,
            uint64_t *)
HMR_UNBUILT(hmr_max_pool2d_gather_backward, hmr_context_t, const hmr_tensor_desc *, const hmr_tensor_desc *,
            const hmr_tensor_desc *, const int64_t *)
HMR_UNBUILT(hmr_adaptive_avg_pool2d, hmr_context_t, const hmr_tensor_desc *, const hmr_tensor_desc *)
HMR_UNBUILT(hmr_adaptive_avg_pool2d_backward, hmr_context_t, const hmr_tensor_desc *, const hmr_tensor_desc *)
HMR_UNBUILT(hmr_unfold_backward, hmr_context_t, const hmr_tensor_desc *, const hmr_tensor_desc *, int32_t, int64_t,
            int64_t)
HMR_UNBUILT(hmr_gemm_fold, hmr_gemm_desc *)
HMR_UNBUILT(hmr_gemm_select, const hmr_gemm_desc *, int32_t *, int32_t *)
HMR_UNBUILT(hmr_gemm_path_name, int32_t, const char **)
HMR_UNBUILT(hmr_gemm_workspace, const hmr_gemm_desc *, int32_t, int64_t *)
HMR_UNBUILT(hmr_gemm, hmr_context_t, const hmr_gemm_desc *, int32_t, void *, int64_t)
HMR_UNBUILT(hmr_test_pool_candidates, const int64_t *, int64_t, int64_t, int64_t, int64_t, int64_t *)

void hmr_test_wide_pool(int32_t) {}
void hmr_test_force_gemm_path(int32_t) {}

}  // extern "C"
