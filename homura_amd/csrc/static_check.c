/*
 * A plain C program linked STATICALLY against libhomura_rocm.a, the way homura's Rust crate links it
 * (ref: build.rs:60-70: the archive, then amdhip64 and stdc++). It shows that the single relocatable
 * object of the archive resolves every call through the hmr_* symbols alone and that its device code
 * is registered with the HIP runtime when the program starts.
 *
 *   static_check          layout and build facts only; touches no device
 *   static_check gpu      also creates a context and runs fill, add and a column sum on device 0
 */
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "homura_rocm.h"

#define CHECK(call)                                                                  \
    do {                                                                             \
        hmr_status s_ = (call);                                                      \
        if (s_ != HMR_OK) {                                                          \
            fprintf(stderr, "%s -> %d: %s\n", #call, (int)s_, hmr_last_error());     \
            return 1;                                                                \
        }                                                                            \
    } while (0)

static hmr_tensor_desc matrix(void *data, int32_t dtype, int64_t rows, int64_t cols, int64_t row_stride,
                              int64_t col_stride) {
    hmr_tensor_desc d;
    memset(&d, 0, sizeof d);
    d.data = data;
    d.dtype = dtype;
    d.ndim = 2;
    d.sizes[0] = rows;
    d.sizes[1] = cols;
    d.strides[0] = row_stride;
    d.strides[1] = col_stride;
    return d;
}

static int run_on_gpu(void) {
    enum { ROWS = 512, COLS = 256 };
    hmr_context_t ctx = NULL;
    CHECK(hmr_context_create(0, &ctx));
    void *a = NULL, *b = NULL, *sums = NULL, *work = NULL;
    CHECK(hmr_malloc(0, ROWS * COLS * 4, &a));
    CHECK(hmr_malloc(0, ROWS * COLS * 4, &b));
    CHECK(hmr_malloc(0, COLS * 4, &sums));
    hmr_tensor_desc da = matrix(a, HMR_F32, ROWS, COLS, COLS, 1);
    hmr_tensor_desc db = matrix(b, HMR_F32, ROWS, COLS, COLS, 1);
    const float one_and_half = 1.5f, quarter = 0.25f;
    uint32_t bits = 0;
    memcpy(&bits, &one_and_half, 4);
    CHECK(hmr_fill(ctx, &da, bits));
    memcpy(&bits, &quarter, 4);
    CHECK(hmr_fill(ctx, &db, bits));
    CHECK(hmr_binary(ctx, HMR_BINARY_ADD, &db, &da, &db)); /* b = a + b = 1.75, in place */
    /* Column sums of b: kept = the columns, reduced = the rows, both with the source's strides. */
    hmr_tensor_desc kept, red, out;
    memset(&kept, 0, sizeof kept);
    kept.data = b;
    kept.dtype = HMR_F32;
    kept.ndim = 1;
    kept.sizes[0] = COLS;
    kept.strides[0] = 1;
    red = kept;
    red.sizes[0] = ROWS;
    red.strides[0] = COLS;
    out = kept;
    out.data = sums;
    int64_t bytes = 0;
    CHECK(hmr_reduce_workspace(&kept, &red, 0, &bytes));
    if (bytes > 0) CHECK(hmr_malloc(0, (uint64_t)bytes, &work));
    CHECK(hmr_reduce(ctx, HMR_REDUCE_SUM, &out, &kept, &red, work, bytes));
    float host[COLS];
    CHECK(hmr_copy_to_host(ctx, host, sums, sizeof host));
    for (int c = 0; c < COLS; ++c) {
        if (host[c] != 1.75f * ROWS) {
            fprintf(stderr, "column %d sums to %g, expected %g\n", c, host[c], 1.75 * ROWS);
            return 1;
        }
    }
    if (work) CHECK(hmr_free(0, work));
    CHECK(hmr_free(0, sums));
    CHECK(hmr_free(0, b));
    CHECK(hmr_free(0, a));
    CHECK(hmr_context_destroy(ctx));
    printf("gpu: fill, add and column sums of [%d, %d] f32 are exact\n", ROWS, COLS);
    return 0;
}

int main(int argc, char **argv) {
    hmr_abi_info info;
    hmr_abi_check(&info);
    if (info.desc_size != sizeof(hmr_tensor_desc) || info.max_dims != HMR_MAX_DIMS ||
        info.abi_info_size != sizeof(hmr_abi_info)) {
        fprintf(stderr, "hmr_abi_check disagrees with the header\n");
        return 1;
    }
    printf("archs %s, desc %u bytes, max dims %d\n", hmr_built_archs(), (unsigned)info.desc_size, (int)info.max_dims);
    if (hmr_test_fail("static check") != HMR_INVALID || strcmp(hmr_last_error(), "static check") != 0) {
        fprintf(stderr, "the error channel does not hold the message\n");
        return 1;
    }
    if (argc > 1 && strcmp(argv[1], "gpu") == 0) return run_on_gpu();
    return 0;
}
