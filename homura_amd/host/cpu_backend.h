/*
 * cpu_backend.h -- the kernel interface a CPU backend offers to the host layer's dispatch.
 *
 * homura dispatches every tensor kernel on the device of its operands
 * (ref: src/backend/mod.rs:44-55, 298-534): `Device::Cpu` goes to `cpu::<kernel>`,
 * `Device::Rocm(i)` to `rocm::<kernel>`. This library ships the ROCm arm only. The CPU arm is a
 * table of function pointers with the signatures of the reference's CPU kernels
 * (ref: src/backend/cpu/mod.rs:28-38) that a process may register at run time; without one,
 * every kernel on a CPU tensor fails with "no CPU backend is registered". Nothing in this
 * package provides such a table.
 *
 * Tensors are described un-merged, exactly as the CPU kernels of the reference receive them
 * (shape + strides + offset in elements); the backend does its own loop-nest planning.
 */
#ifndef HOMURA_CPU_BACKEND_H
#define HOMURA_CPU_BACKEND_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct hcb_tensor {
    void *data;             /* first byte of the storage */
    int64_t offset;         /* of element (0,..,0), in elements */
    int32_t dtype;          /* HMR_BOOL .. HMR_F64 */
    int32_t ndim;
    const int64_t *shape;   /* ndim entries */
    const int64_t *strides; /* ndim entries, in elements, >= 0 */
} hcb_tensor;

/* homura's Scalar (ref: src/dtype.rs:285-293). */
#define HCB_SCALAR_BOOL 0
#define HCB_SCALAR_INT 1
#define HCB_SCALAR_FLOAT 2
typedef struct hcb_scalar {
    int32_t kind;
    int32_t reserved;
    int64_t i; /* value for BOOL (0/1) and INT */
    double f;  /* value for FLOAT */
} hcb_scalar;

/*
 * Every kernel returns 0, or nonzero where the reference's CPU kernel would panic; the text of
 * that panic is then available from last_error() until the thread's next call.
 * All operands of one call have the same shape (inputs already expanded by the caller).
 */
typedef struct hcb_backend {
    const char *name;
    const char *(*last_error)(void);
    /* ref: src/backend/cpu/mod.rs:315-332 */
    int (*copy)(const hcb_tensor *dst, const hcb_tensor *src);
    int (*fill)(const hcb_tensor *dst, hcb_scalar value);
    /* ref: src/backend/cpu/mod.rs:336-507 */
    int (*unary)(int32_t op, const hcb_tensor *out, const hcb_tensor *src);
    int (*binary)(int32_t op, const hcb_tensor *out, const hcb_tensor *a, const hcb_tensor *b);
    int (*binary_constant)(int32_t op, const hcb_tensor *out, const hcb_tensor *a,
                           hcb_scalar value, int32_t constant_first);
    int (*binary_scalar)(int32_t op, const hcb_tensor *out, const hcb_tensor *a, double s,
                         int32_t scalar_first);
    /* ref: src/backend/cpu/mod.rs:573-600; a NULL branch is the constant beside it */
    int (*where_)(const hcb_tensor *out, const hcb_tensor *cond, const hcb_tensor *x,
                  const hcb_tensor *y);
    int (*where_constant)(const hcb_tensor *out, const hcb_tensor *cond, const hcb_tensor *x,
                          hcb_scalar x_value, const hcb_tensor *y, hcb_scalar y_value);
    /* ref: src/backend/cpu/reduce.rs:92-225; mask has src->ndim entries (1 = reduced) */
    int (*reduce)(int32_t op, const hcb_tensor *out, const hcb_tensor *src, const uint8_t *mask);
    int (*var)(const hcb_tensor *out, const hcb_tensor *src, const uint8_t *mask,
               double correction, int32_t take_sqrt);
    int (*arg_reduce)(const hcb_tensor *values, const hcb_tensor *indices, const hcb_tensor *src,
                      int32_t dim, int32_t is_max);
    /* ref: src/backend/cpu/misc.rs:15-51 */
    int (*softmax)(const hcb_tensor *out, const hcb_tensor *src, int32_t dim, int32_t log);
    /* ref: src/backend/cpu/mod.rs:509-569; kind 0 ScaledAdd(alpha), 1 Lerp(weight), 2 Addcmul(value),
     * 3 Addcdiv(value), with the caller's f64 scalar; c is NULL for kinds 0 and 1 */
    int (*fused)(int32_t kind, double scalar, const hcb_tensor *out, const hcb_tensor *a,
                 const hcb_tensor *b, const hcb_tensor *c);
    /* ref: src/backend/cpu/misc.rs:347-411; flip's mask has src->ndim entries (1 = reversed) */
    int (*triangle)(const hcb_tensor *out, const hcb_tensor *src, int64_t diagonal, int32_t upper);
    int (*flip)(const hcb_tensor *out, const hcb_tensor *src, const uint8_t *mask);
    /* ref: src/backend/cpu/linalg.rs:224-388; out is [n, m], v1 [n], v2 [m], input a view of [n, m]
     * that is read only when beta isn't zero; alpha and beta are values of the dtype */
    int (*addr)(const hcb_tensor *out, const hcb_tensor *v1, const hcb_tensor *v2,
                const hcb_tensor *input, hcb_scalar alpha, hcb_scalar beta);
    /* ref: src/backend/cpu/reduce.rs:281-324; floating point operands of one shape and dtype */
    int (*exclusive_cumprod)(const hcb_tensor *out, const hcb_tensor *src, int32_t dim,
                             int32_t reverse);
    /* ref: src/ops/random.rs:29-266: the samples of the Philox blocks from `offset` on under `seed`
     * into a flat contiguous tensor (floats; I64 for random_int). random_int is one batch of the
     * rejection sampling over `blocks` blocks and reports how many words it accepted. */
    int (*random_uniform)(const hcb_tensor *out, uint64_t seed, uint64_t offset, double from,
                          double to);
    int (*random_normal)(const hcb_tensor *out, uint64_t seed, uint64_t offset, double mean,
                         double std);
    int (*random_int)(const hcb_tensor *out, uint64_t seed, uint64_t offset, uint64_t blocks,
                      int64_t low, uint64_t range, uint64_t threshold, uint64_t *accepted);
    /* ref: src/backend/cpu/misc.rs:53-127, 213-345. `index` is I32 or I64; `bounds`: 0 the positions
     * are valid, 1 none may be negative, 2 negative ones count from the end; the first position
     * out of range fails the call with "index {v} is out of bounds for dimension {dim} with size
     * {size}". index_add and scatter_add add into a contiguous `out` that shares no memory with
     * `src`, each element summed in f64 (wrapping i64 for integers) in row-major order of the
     * index and rounded once. */
    int (*index_select)(const hcb_tensor *out, const hcb_tensor *src, int32_t dim,
                        const hcb_tensor *index, int32_t bounds);
    int (*gather)(const hcb_tensor *out, const hcb_tensor *src, int32_t dim,
                  const hcb_tensor *index);
    int (*index_add)(const hcb_tensor *out, int32_t dim, const hcb_tensor *index,
                     const hcb_tensor *src, int32_t bounds);
    int (*scatter_add)(const hcb_tensor *out, int32_t dim, const hcb_tensor *index,
                       const hcb_tensor *src);
    /* ref: src/backend/cpu/misc.rs:104-126. Slice i of src along dim is copied to slice index[i]
     * (valid positions) of out, in order: the last of repeated positions wins. */
    int (*index_overwrite)(const hcb_tensor *out, int32_t dim, const hcb_tensor *index,
                           const hcb_tensor *src);
    /* ref: src/backend/cpu/misc.rs:128-148. *count = the number of true elements of the BOOL mask;
     * with `out` (I64, contiguous, the mask's rank x that number) coordinate d of the k-th true
     * element in row-major order goes to out[d][k]. */
    int (*mask_coordinates)(const hcb_tensor *mask, const hcb_tensor *out, int64_t *count);
    /* ref: src/backend/cpu/misc.rs:150-203. The `n` indices (I32 or I64) are checked in order to lie
     * in -sizes[k]..sizes[k]: the first value out of range is left in (*bad_index, *bad_value) and
     * nothing is written; otherwise *bad_index = -1 and, with `out` (I64, contiguous, the shape the
     * indices broadcast to), every element gets its row-major position in the subspace of
     * `sizes`, negative coordinates counting from the end. */
    int (*index_positions)(const hcb_tensor *out, int32_t n, const hcb_tensor *const *coords,
                           const int64_t *sizes, int32_t *bad_index, int64_t *bad_value);
} hcb_backend;

#ifdef __cplusplus
}
#endif

#endif /* HOMURA_CPU_BACKEND_H */
