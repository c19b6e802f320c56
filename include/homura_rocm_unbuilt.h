/*
 * homura_rocm_unbuilt.h -- entry points of the reference's C ABI that belong to kernel families
 * this library does not implement (pooling, unfold, matrix products). They are exported so that
 * the reference crate's 77 `extern "C"` declarations (ref: src/backend/rocm/ffi.rs) all resolve
 * at link time; each one fails with HMR_INVALID and the message
 * "<name>: not built in this library". The size queries among them (`*_workspace`) fail the same
 * way, so a caller never allocates for a kernel that cannot run.
 *
 * Signatures follow ref: csrc/homura_rocm.h at the line given beside each declaration.
 */
#ifndef HOMURA_ROCM_UNBUILT_H
#define HOMURA_ROCM_UNBUILT_H

#include "homura_rocm.h"

#ifdef __cplusplus
extern "C" {
#endif

/* ref :407-414 (the backward of max pooling through sorted positions) */
hmr_status hmr_max_pool2d_backward_workspace(int64_t n, int64_t *bytes);
hmr_status hmr_max_pool2d_backward(hmr_context_t ctx, const hmr_tensor_desc *out,
                                   const hmr_tensor_desc *grad, const hmr_tensor_desc *indices,
                                   void *workspace, int64_t workspace_bytes);

/* ref :434-466 (pooling) */
hmr_status hmr_max_pool2d(hmr_context_t ctx, const hmr_tensor_desc *out,
                          const hmr_tensor_desc *indices, const hmr_tensor_desc *input,
                          const int64_t *geometry);
hmr_status hmr_max_pool2d_check(hmr_context_t ctx, const hmr_tensor_desc *indices,
                                int64_t height, int64_t width, const int64_t *geometry,
                                uint64_t *slot);
hmr_status hmr_max_pool2d_gather_backward(hmr_context_t ctx, const hmr_tensor_desc *out,
                                          const hmr_tensor_desc *grad,
                                          const hmr_tensor_desc *indices,
                                          const int64_t *geometry);
hmr_status hmr_adaptive_avg_pool2d(hmr_context_t ctx, const hmr_tensor_desc *out,
                                   const hmr_tensor_desc *input);
hmr_status hmr_adaptive_avg_pool2d_backward(hmr_context_t ctx, const hmr_tensor_desc *out,
                                            const hmr_tensor_desc *grad);
hmr_status hmr_unfold_backward(hmr_context_t ctx, const hmr_tensor_desc *out,
                               const hmr_tensor_desc *grad, int32_t dim, int64_t size,
                               int64_t step);

/* ref :485-510. Kept only so hmr_abi_check can report its size and alignment (256, 8). */
typedef struct hmr_gemm_desc {
    int32_t dtype;
    int32_t sum_batches;
    int32_t scaled;
    int32_t reads_input;
    int64_t batch, m, n, k;
    const void *a;
    const void *b;
    const void *c;
    void *out;
    int64_t a_strides[3];
    int64_t b_strides[3];
    int64_t c_strides[3];
    int64_t out_strides[3];
    double alpha;
    double beta;
    int64_t alpha_int;
    int64_t beta_int;
} hmr_gemm_desc;

/* ref :569-587 (matrix products) */
hmr_status hmr_gemm_fold(hmr_gemm_desc *desc);
hmr_status hmr_gemm_select(const hmr_gemm_desc *desc, int32_t *path, int32_t *layout);
hmr_status hmr_gemm_path_name(int32_t path, const char **name);
hmr_status hmr_gemm_workspace(const hmr_gemm_desc *desc, int32_t path, int64_t *bytes);
hmr_status hmr_gemm(hmr_context_t ctx, const hmr_gemm_desc *desc, int32_t path, void *workspace,
                    int64_t workspace_bytes);

/* ref :657-662 (test hooks of the families above) */
void hmr_test_wide_pool(int32_t on);
void hmr_test_force_gemm_path(int32_t path);
hmr_status hmr_test_pool_candidates(const int64_t *geometry, int64_t height, int64_t width,
                                    int64_t out_h, int64_t out_w, int64_t *count);

#ifdef __cplusplus
}
#endif

#endif /* HOMURA_ROCM_UNBUILT_H */
