/*
 * homura_rocm.h -- C ABI of the gfx950 (MI355X, CDNA4, wave64) build of homura's ROCm layer.
 *
 * This header is a drop-in for the reference's csrc/homura_rocm.h for the tensor elementwise,
 * broadcast, copy/convert, reduction and softmax entry points, plus the plumbing those need
 * (contexts, memory, error text). Every declaration names the reference declaration it replaces
 * as `ref: csrc/homura_rocm.h:<line>`; signatures, struct layouts and enumerator values are the
 * same, so the Rust bindings in src/backend/rocm/ffi.rs bind to this library unchanged.
 *
 * Calling conventions (ref: csrc/homura_rocm.h:1-15):
 *  - plain C, <stdint.h>/<stddef.h> only;
 *  - every entry point returns an hmr_status; after a failure hmr_last_error() holds a message
 *    that belongs to the calling thread and lives until that thread calls the library again;
 *  - no C++ exception leaves the library;
 *  - an entry point that uses a device makes it current for the calling thread and puts the
 *    previous device back before it returns;
 *  - enumerations travel as int32_t.
 *
 * Entry points of the reference that belong to other kernel families (gemm, pooling, convolution
 * windows, the rest of indexing ...) are declared in homura_rocm_unbuilt.h and exported as
 * stubs that fail with HMR_INVALID, so that the reference crate still links.
 */
#ifndef HOMURA_ROCM_H
#define HOMURA_ROCM_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- status ------------------------------------------------- ref: csrc/homura_rocm.h:26-40 */
#define HMR_OK 0
#define HMR_OUT_OF_MEMORY 1 /* a device allocation found no memory */
#define HMR_INVALID 2       /* bad argument, unsupported GPU, unsupported dtype/op pair */
#define HMR_HIP_ERROR 3     /* the HIP runtime reported an error */
#define HMR_INTERNAL_ERROR 4 /* a failure inside the library (e.g. a C++ exception) */

typedef int32_t hmr_status;

/* Text of the calling thread's most recent failure ("" when it has had none). */
const char *hmr_last_error(void);

/* ---- devices ------------------------------------------------ ref: csrc/homura_rocm.h:42-64 */
#define HMR_NAME_LEN 256
#define HMR_ARCH_LEN 64

typedef struct hmr_device_properties {
    char name[HMR_NAME_LEN]; /* marketing name */
    char arch[HMR_ARCH_LEN]; /* "gfx950": gcnArchName without the ":sramecc+:xnack-" features */
    /* hipDeviceProp_t::multiProcessorCount. On CDNA this IS the number of compute units (256
     * on MI355X); the reference's doubling for RDNA work-group processors does not apply. */
    int32_t multiprocessor_count;
    int32_t warp_size; /* 64 on gfx950 */
    uint64_t total_memory;
} hmr_device_properties;

/* Visible devices; 0 with HMR_OK when there is no device or no driver. */
hmr_status hmr_device_count(int32_t *count);
hmr_status hmr_device_properties_get(int32_t device, hmr_device_properties *out);
hmr_status hmr_mem_get_info(int32_t device, uint64_t *free_bytes, uint64_t *total_bytes);

/* ---- contexts ----------------------------------------------- ref: csrc/homura_rocm.h:66-79 */
/* One per device: owns the non-blocking stream every kernel of that device is queued on. */
typedef struct hmr_context *hmr_context_t;

/* Fails with HMR_INVALID unless the GPU is one the library was built for (gfx950) and runs
 * 64-lane wavefronts; then creates the stream and runs a probe kernel on it. Leaves nothing
 * allocated on failure. */
hmr_status hmr_context_create(int32_t device, hmr_context_t *out);
hmr_status hmr_context_destroy(hmr_context_t ctx);
/* Blocks until the context's stream is idle. */
hmr_status hmr_context_synchronize(hmr_context_t ctx);

/* ---- memory ------------------------------------------------- ref: csrc/homura_rocm.h:81-100 */
/* hipMalloc / hipFree on `device`; running out of memory is HMR_OUT_OF_MEMORY and is not left
 * behind as HIP's sticky last error. The caller's caching allocator sits on top of these. */
hmr_status hmr_malloc(int32_t device, uint64_t nbytes, void **out);
hmr_status hmr_free(int32_t device, void *ptr);
/* Stream-ordered byte fill. */
hmr_status hmr_memset(hmr_context_t ctx, void *ptr, uint8_t value, uint64_t nbytes);
/* Stream-ordered copies to/from pageable host memory; they return once the bytes have moved. */
hmr_status hmr_copy_to_host(hmr_context_t ctx, void *dst, const void *src, uint64_t nbytes);
hmr_status hmr_copy_from_host(hmr_context_t ctx, void *dst, const void *src, uint64_t nbytes);

/* ---- element types ------------------------------------------ ref: csrc/homura_rocm.h:102-113 */
/* Numbered as homura's DType. BOOL is one byte holding 0 or 1; F16/BF16 are raw 16-bit patterns. */
#define HMR_BOOL 0
#define HMR_U8 1
#define HMR_I8 2
#define HMR_I16 3
#define HMR_I32 4
#define HMR_I64 5
#define HMR_F16 6
#define HMR_BF16 7
#define HMR_F32 8
#define HMR_F64 9

/* ---- tensor descriptions ------------------------------------ ref: csrc/homura_rocm.h:115-130 */
#define HMR_MAX_DIMS 25

/* Element (i_0 .. i_{ndim-1}) lives at data[offset + sum_k i_k * strides[k]], counted in
 * elements of `dtype`. ndim == 0 describes one element. The caller merges dimensions first
 * (size-1 dims dropped, neighbours that are contiguous in every operand joined). 424 bytes. */
typedef struct hmr_tensor_desc {
    void *data;
    int64_t offset;
    int32_t dtype;
    int32_t ndim;
    int64_t sizes[HMR_MAX_DIMS];
    int64_t strides[HMR_MAX_DIMS];
} hmr_tensor_desc;

/* ---- copy / convert / fill ---------------------------------- ref: csrc/homura_rocm.h:132-146 */
/* dst[i] = cast(src[i]) with homura's Element::to_element rules (src/dtype.rs:171-277): float
 * sources go through f64; halves are rounded through f32; float->int truncates, saturates to
 * i64 and wraps; NaN payloads follow the CPU's conversions. Same ndim/sizes; src strides may
 * be 0. Equal dtypes move the bytes. */
hmr_status hmr_copy(hmr_context_t ctx, const hmr_tensor_desc *dst, const hmr_tensor_desc *src);
/* Every element of dst = the element whose little-endian bytes are the low bytes of `bits`. */
hmr_status hmr_fill(hmr_context_t ctx, const hmr_tensor_desc *dst, uint64_t bits);
/* hipMemcpyAsync device->device of non-overlapping ranges on the context's device. */
hmr_status hmr_copy_device(hmr_context_t ctx, void *dst, const void *src, uint64_t nbytes);

/* ---- elementwise -------------------------------------------- ref: csrc/homura_rocm.h:148-263 */
/*
 * Results are those of homura's CPU backend (src/backend/cpu/mod.rs:336-600): F16/BF16/F32 are
 * computed in f32 and F64 in f64 with one rounding to the dtype, integers wrap. Operands share
 * ndim and sizes; input strides may be 0; the output's elements are distinct and either do not
 * overlap an input or are that input (in place). HMR_INVALID for an op the dtype has no rule for.
 */
#define HMR_UNARY_NEG 0
#define HMR_UNARY_ABS 1
#define HMR_UNARY_SIGN 2
#define HMR_UNARY_RELU 3
#define HMR_UNARY_EXP 4
#define HMR_UNARY_LOG 5
#define HMR_UNARY_SQRT 6
#define HMR_UNARY_RSQRT 7
#define HMR_UNARY_RECIPROCAL 8
#define HMR_UNARY_SIN 9
#define HMR_UNARY_COS 10
#define HMR_UNARY_ERF 11
#define HMR_UNARY_TANH 12
#define HMR_UNARY_SIGMOID 13
#define HMR_UNARY_LOG_SIGMOID 14
#define HMR_UNARY_SILU 15
#define HMR_UNARY_GELU 16
#define HMR_UNARY_GELU_TANH 17
#define HMR_UNARY_LOGICAL_NOT 18

#define HMR_BINARY_ADD 0
#define HMR_BINARY_SUB 1
#define HMR_BINARY_MUL 2
#define HMR_BINARY_DIV 3
#define HMR_BINARY_POW 4
#define HMR_BINARY_MAXIMUM 5
#define HMR_BINARY_MINIMUM 6
#define HMR_BINARY_GREATER 7
#define HMR_BINARY_GREATER_EQUAL 8
#define HMR_BINARY_LESS 9
#define HMR_BINARY_LESS_EQUAL 10
#define HMR_BINARY_EQUAL 11
#define HMR_BINARY_NOT_EQUAL 12
#define HMR_BINARY_LOGICAL_AND 13
#define HMR_BINARY_LOGICAL_OR 14
/* Extension (the reference has no bitwise op, ref: src/ops/mod.rs:68-85): two's-complement `&`
 * on integer dtypes, logical and on BOOL; floats are HMR_INVALID. Appended, nothing renumbered. */
#define HMR_BINARY_BITWISE_AND 15

/* ref :202  out = op(src). LOGICAL_NOT writes BOOL, everything else src's dtype. */
hmr_status hmr_unary(hmr_context_t ctx, int32_t op, const hmr_tensor_desc *out,
                     const hmr_tensor_desc *src);

/* ref :206  out = op(a, b). Comparisons and logical ops write BOOL.
 * Extension: when a and b are floating point dtypes that differ, each is first converted
 * (exactly) to out's dtype, which must be their promotion; this folds the reference's separate
 * cast kernel (ref: src/ops/mod.rs:177-195) into the op and yields the same bits. */
hmr_status hmr_binary(hmr_context_t ctx, int32_t op, const hmr_tensor_desc *out,
                      const hmr_tensor_desc *a, const hmr_tensor_desc *b);

/* ref :212  hmr_binary with the other operand equal to the constant whose bytes are the low
 * bytes of `bits` (an element of a's dtype); op(c, a) when constant_first. */
hmr_status hmr_binary_constant(hmr_context_t ctx, int32_t op, const hmr_tensor_desc *out,
                               const hmr_tensor_desc *a, uint64_t bits, int32_t constant_first);

/* ref :217  MUL and DIV only, float `a`: a*s, a/s or (scalar_first) s/a with `s` rounded to the
 * computation type, not to the dtype (f16/bf16 keep an f32 scalar). */
hmr_status hmr_binary_scalar(hmr_context_t ctx, int32_t op, const hmr_tensor_desc *out,
                             const hmr_tensor_desc *a, double s, int32_t scalar_first);

/* ref :247  out = cond ? x : y, cond BOOL, x and y of out's dtype. */
hmr_status hmr_where(hmr_context_t ctx, const hmr_tensor_desc *out, const hmr_tensor_desc *cond,
                     const hmr_tensor_desc *x, const hmr_tensor_desc *y);

/* ref :253  hmr_where where a NULL branch stands for the constant x_bits / y_bits. */
hmr_status hmr_where_constant(hmr_context_t ctx, const hmr_tensor_desc *out,
                              const hmr_tensor_desc *cond, const hmr_tensor_desc *x,
                              uint64_t x_bits, const hmr_tensor_desc *y, uint64_t y_bits);

/* ---- fused optimiser steps, addr, triangle, flip ------------- ref: csrc/homura_rocm.h:195-263 */
#define HMR_FUSED_SCALED_ADD 0
#define HMR_FUSED_LERP 1
#define HMR_FUSED_ADDCMUL 2
#define HMR_FUSED_ADDCDIV 3

/* ref :221-230  cpu::fused (src/backend/cpu/mod.rs:509-569): floating point operands of one dtype,
 * one rounding to it; `c` is NULL for SCALED_ADD and LERP. `coefficient` is already in the
 * computation type (f32 for F16/BF16/F32): alpha rounded to the dtype first, the Lerp coefficient
 * (weight, or weight - 1 when `small` is 0), or value.
 *   SCALED_ADD fma(b, coefficient, a)          LERP    fma(coefficient, b - a, small ? a : b)
 *   ADDCMUL    fma(coefficient * b, c, a)      ADDCDIV a + coefficient * b / c */
hmr_status hmr_fused(hmr_context_t ctx, int32_t op, const hmr_tensor_desc *out,
                     const hmr_tensor_desc *a, const hmr_tensor_desc *b,
                     const hmr_tensor_desc *c, double coefficient, int32_t small);

/* ref :232-244  cpu::addr (src/backend/cpu/linalg.rs:224-388): out[i][j] = beta * input[i][j] +
 * alpha * v1[i] * v2[j] for every dtype. All four descriptions have the output's two dimensions
 * [n, m]: v1 with stride 0 along the columns, v2 along the rows, the input broadcast as needed;
 * `input` may be NULL when beta is zero (it isn't read then).
 *   floats (coefficients already rounded to the dtype, in `alpha` and `beta`): a = alpha * v1[i]
 *     (skipped for alpha == 1), p = a * v2[j], out = p or (beta == 1 ? c : beta * c) + p, each step
 *     in the computation type and rounded to the dtype;
 *   integers (`alpha_int`, `beta_int`): wrapping, alpha * (v1[i] * v2[j]) + beta * c;
 *   Bool (`alpha_int`, `beta_int` 0 or 1): (v1[i] and alpha and v2[j]) or (beta and c). */
hmr_status hmr_addr(hmr_context_t ctx, const hmr_tensor_desc *out, const hmr_tensor_desc *v1,
                    const hmr_tensor_desc *v2, const hmr_tensor_desc *input, double alpha,
                    double beta, int64_t alpha_int, int64_t beta_int);

/* ref :257-260  cpu::triangle (src/backend/cpu/misc.rs:347-381): out = src where the column minus
 * the row index (the last two dimensions, ndim >= 2) is at least (upper) or at most `diagonal`,
 * else 0. Any dtype, one for both. */
hmr_status hmr_triangle(hmr_context_t ctx, const hmr_tensor_desc *out,
                        const hmr_tensor_desc *src, int64_t diagonal, int32_t upper);

/* ref :262-263  cpu::flip (src/backend/cpu/misc.rs:384-411): out = src for one dtype, where src's
 * strides may be negative (reversed dimensions, offset at the last element of each). */
hmr_status hmr_flip(hmr_context_t ctx, const hmr_tensor_desc *out, const hmr_tensor_desc *src);

/* ---- reductions --------------------------------------------- ref: csrc/homura_rocm.h:297-346 */
/*
 * `kept`: the kept dimensions with the SOURCE's strides, data, offset, dtype; `red`: the reduced
 * dimensions with the source's strides (same dtype). Outputs are contiguous over kept's sizes.
 * The fold order depends only on sizes and strides, so results repeat from run to run. Plans
 * that cut the reduced range across workgroups stage partial results in `workspace`, whose size
 * hmr_reduce_workspace reports (var = 1 for hmr_var); NULL is fine when that is 0.
 */
#define HMR_REDUCE_SUM 0
#define HMR_REDUCE_PROD 1
#define HMR_REDUCE_MEAN 2
#define HMR_REDUCE_MAX 3
#define HMR_REDUCE_MIN 4
#define HMR_REDUCE_ALL 5
#define HMR_REDUCE_ANY 6

/* ref :315 */
hmr_status hmr_reduce_workspace(const hmr_tensor_desc *kept, const hmr_tensor_desc *red,
                                int32_t var, int64_t *bytes);

/* ref :321  cpu::reduce (src/backend/cpu/reduce.rs:92-131): float SUM/PROD/MEAN accumulate in
 * f64; integer and bool SUM/PROD wrap in i64 and write I64; MAX/MIN keep the dtype (first NaN
 * wins, then the first of equals) and need a nonempty range; ALL/ANY write BOOL (U8 for U8). */
hmr_status hmr_reduce(hmr_context_t ctx, int32_t op, const hmr_tensor_desc *out,
                      const hmr_tensor_desc *kept, const hmr_tensor_desc *red, void *workspace,
                      int64_t workspace_bytes);

/* No counterpart in the reference. hmr_reduce for callers that cannot allocate device memory (code
 * under HIP graph capture, serving loops, harnesses that forbid hipMalloc) and so have no workspace
 * to pass: the partial results go to HMR_REDUCE_STATIC_BYTES of device memory that the library's
 * code object holds on every GPU it runs on, bound when the context is created. Same results as
 * hmr_reduce, bit for bit. HMR_INVALID, with nothing queued, when the reduction's plan needs more
 * than that (hmr_reduce_workspace reports the need). Allocates nothing. A GPU's block belongs to one
 * context at a time - the first that stages partial results in it, until that context is destroyed -
 * and another context of the same GPU is refused with HMR_INVALID (two contexts have two streams,
 * whose kernels would overwrite each other's partial results). Calls on the owning context run on its
 * one stream, in order; as for every entry point, one thread at a time calls into a context. */
#define HMR_REDUCE_STATIC_BYTES (8 * 1024 * 1024)
hmr_status hmr_reduce_static(hmr_context_t ctx, int32_t op, const hmr_tensor_desc *out,
                             const hmr_tensor_desc *kept, const hmr_tensor_desc *red);

/* ref :327  cpu::var (src/backend/cpu/reduce.rs:135-170): f64 variance about the f64 mean,
 * divided by max(0, n - correction); NaN for n == 0; sqrt of it with take_sqrt. */
hmr_status hmr_var(hmr_context_t ctx, const hmr_tensor_desc *out, const hmr_tensor_desc *kept,
                   const hmr_tensor_desc *red, double correction, int32_t take_sqrt,
                   void *workspace, int64_t workspace_bytes);

/* ref :333  cpu::arg_reduce (src/backend/cpu/reduce.rs:175-225): I64 index along the single
 * reduced dimension of the max (min) and, when `values` is not NULL, the value itself. */
hmr_status hmr_arg_reduce(hmr_context_t ctx, const hmr_tensor_desc *values,
                          const hmr_tensor_desc *indices, const hmr_tensor_desc *kept,
                          const hmr_tensor_desc *red, int32_t is_max, void *workspace,
                          int64_t workspace_bytes);

/* ref :341-346  cpu::softmax (src/backend/cpu/misc.rs:15-51) over rows of n elements:
 * `out_rows` / `src_rows` describe the remaining dimensions, row elements are out_stride /
 * src_stride apart. */
hmr_status hmr_softmax_workspace(const hmr_tensor_desc *src_rows, int64_t n, int64_t src_stride,
                                 int64_t *bytes);
hmr_status hmr_softmax(hmr_context_t ctx, const hmr_tensor_desc *out_rows,
                       const hmr_tensor_desc *src_rows, int64_t n, int64_t out_stride,
                       int64_t src_stride, int32_t log, void *workspace,
                       int64_t workspace_bytes);

/* ref :348-351  cpu::exclusive_cumprod (src/backend/cpu/reduce.rs:281-324) along lines of n
 * elements, described as for hmr_softmax: out[k] = the product of the line's elements before k
 * (after k when `reverse`), 1 for the first (last), accumulated in order in f32 (F16, BF16) or
 * f64 (F32, F64) and rounded to the dtype as it is written. Floating point dtypes, one for both. */
hmr_status hmr_exclusive_cumprod(hmr_context_t ctx, const hmr_tensor_desc *out_lines,
                                 const hmr_tensor_desc *src_lines, int64_t n, int64_t out_stride,
                                 int64_t src_stride, int32_t reverse);

/* ---- random sampling ------------------------------------------ ref: csrc/homura_rocm.h:265-295 */
/* Philox4x32-10 as in src/ops/random.rs:29-91: block n is the counter [n, n >> 32, 0, 0] under the
 * key [seed, seed >> 32]; the caller reserves the blocks of a call (from `offset` on) as the CPU
 * does and advances its generator. `out` is flat and contiguous.
 *
 * ref :276-279  hmr_random_uniform: from + u * (to - from) in f64 for a float `out`, u from 53
 * bits (two words, two elements per block) for F64 and from the dtype's significand bits (one
 * word per element, four per block) otherwise, rounded to the dtype; a result that rounds to `to`
 * (with from < to) becomes `from`. hmr_random_normal: Box-Muller in f64, two elements per block
 * (cosine, then sine), rounded to the dtype. */
hmr_status hmr_random_uniform(hmr_context_t ctx, const hmr_tensor_desc *out, uint64_t seed,
                              uint64_t offset, double from, double to);
hmr_status hmr_random_normal(hmr_context_t ctx, const hmr_tensor_desc *out, uint64_t seed,
                             uint64_t offset, double mean, double std);

/* The Philox blocks of one tile of hmr_random_int. */
#define HMR_RANDOM_INT_TILE 256

/* ref :284-295  One batch of the CPU's integer rejection sampling (sample_int,
 * src/ops/random.rs:228-258): the 64-bit words of `blocks` blocks from `offset` on, two per block
 * in the order [w0 w1] then [w2 w3]; the words >= `threshold`, in that order, become
 * low + word % range (wrapping) and fill the I64 `out` until it is full, the rest are dropped.
 * With threshold 0 every word is taken and `workspace` may be NULL. Otherwise `workspace` holds
 * 2 * tiles + 1 64-bit words of device memory, tiles = ceil(blocks / HMR_RANDOM_INT_TILE), and
 * the batch's number of words >= threshold (which may exceed out's elements) is left in its last
 * word. */
hmr_status hmr_random_int(hmr_context_t ctx, const hmr_tensor_desc *out, uint64_t seed,
                          uint64_t offset, uint64_t blocks, int64_t low, uint64_t range,
                          uint64_t threshold, void *workspace);

/* ---- indexing -------------------------------------------------- ref: csrc/homura_rocm.h:353-404 */
/* Index tensors are I32 or I64; positions are checked before they are used (hmr_index_check, in the
 * same critical section of the caller), so the other entry points take them as valid.
 *
 * ref :358-363  The first element of `index`, in row-major order of its logical positions, that is
 * outside [low, high) and, if has_exempt, not equal to `exempt`: queues writing its position to
 * slot[0] (UINT64_MAX if there is none) and its value to slot[1]. `slot` is two words of device
 * memory. */
hmr_status hmr_index_check(hmr_context_t ctx, const hmr_tensor_desc *index, int64_t low,
                           int64_t high, int32_t has_exempt, int64_t exempt, uint64_t *slot);

/* ref :365-370  cpu::index_select (src/backend/cpu/misc.rs:74-105): out (src's sizes but the 1-D
 * `index`'s length along dim) gets the slices of src along dim at the positions of `index`,
 * negative ones counted from the end if wrap_negative. */
hmr_status hmr_index_select(hmr_context_t ctx, const hmr_tensor_desc *out,
                            const hmr_tensor_desc *src, const hmr_tensor_desc *index, int32_t dim,
                            int32_t wrap_negative);

/* ref :372-375  cpu::gather (misc.rs:313-345): out (index's sizes) gets src at each index position
 * with the coordinate along dim replaced by the index element. */
hmr_status hmr_gather(hmr_context_t ctx, const hmr_tensor_desc *out, const hmr_tensor_desc *src,
                      const hmr_tensor_desc *index, int32_t dim);

/* ref :392-399  cpu::index_add (misc.rs:254-290): slice i of src along dim is added into slice
 * index[i] of out, each element of out summed in f64 (floats; integers wrap in i64, bools are
 * or-ed) in the order of i and rounded once. The workspace has hmr_index_add_workspace bytes for
 * `m` positions (`size`, out's size along dim, bounds them). Here: m < 2^31, size < 2^32. */
hmr_status hmr_index_add_workspace(int64_t m, int64_t size, int64_t *bytes);
hmr_status hmr_index_add(hmr_context_t ctx, const hmr_tensor_desc *out,
                         const hmr_tensor_desc *src, const hmr_tensor_desc *index, int32_t dim,
                         void *workspace, int64_t workspace_bytes);

/* ref :401-408  cpu::scatter_add (misc.rs:292-311): src at each index position is added into out
 * at that position with the coordinate along dim replaced by the index element, summed as
 * hmr_index_add sums, in row-major order of the index positions. `index`, `out` and `src` are
 * described over the index's sizes (out with its own size along dim). The workspace has
 * hmr_scatter_add_workspace bytes for the index's number of elements. Here: fewer than 2^31
 * positions, an output of fewer than 2^32 - 1 elements. */
hmr_status hmr_scatter_add_workspace(int64_t n, int64_t *bytes);
hmr_status hmr_scatter_add(hmr_context_t ctx, const hmr_tensor_desc *out,
                           const hmr_tensor_desc *src, const hmr_tensor_desc *index, int32_t dim,
                           void *workspace, int64_t workspace_bytes);

/* ref :376-380  One indexed dimension of advanced indexing (cpu::index_positions, misc.rs:150-203):
 * out (I64) = (if first) or += coord * stride, the coordinate (I32 or I64) wrapped by `size` when
 * negative; `coord` has out's sizes (broadcast through zero strides). */
hmr_status hmr_index_positions(hmr_context_t ctx, const hmr_tensor_desc *out,
                               const hmr_tensor_desc *coord, int64_t size, int64_t stride,
                               int32_t first);

/* ref :382-389  cpu::index_overwrite (misc.rs:104-126): slice i of src along dim is copied to slice
 * positions[i] of out, the last of repeated positions winning. `positions` is a 1-D tensor of valid
 * positions; out and src are described as for hmr_index_add. The workspace has
 * hmr_index_overwrite_workspace bytes for out's size along dim: an 8-byte word per position of that
 * dimension, whatever the number of slices written. Every call clears all of it first, so a put of a
 * few rows into a dimension of 2^28 positions still asks for 2 GiB and moves 4 GiB. */
hmr_status hmr_index_overwrite_workspace(int64_t size, int64_t *bytes);
hmr_status hmr_index_overwrite(hmr_context_t ctx, const hmr_tensor_desc *out,
                               const hmr_tensor_desc *src, const hmr_tensor_desc *positions,
                               int32_t dim, void *workspace, int64_t workspace_bytes);

/* ref :416-426  cpu::mask_coordinates (misc.rs:128-148) in two calls: hmr_mask_count queues counting
 * the true elements of the BOOL mask (any layout), whose number it leaves at word total_word of the
 * workspace (hmr_mask_workspace bytes for the mask's number of elements: a 64-bit word per tile of
 * 4096 elements and one for the total, and for masks of up to 65 536 tiles a second word per tile);
 * hmr_mask_coordinates then writes coordinate d of the k-th
 * true element, in row-major order, to out[d][k] (I64, the mask's rank x the number). */
hmr_status hmr_mask_workspace(int64_t n, int64_t *bytes, int64_t *total_word);
hmr_status hmr_mask_count(hmr_context_t ctx, const hmr_tensor_desc *mask, void *workspace,
                          int64_t workspace_bytes);
hmr_status hmr_mask_coordinates(hmr_context_t ctx, const hmr_tensor_desc *mask, void *workspace,
                                int64_t workspace_bytes, const hmr_tensor_desc *out);

/* ---- build facts and ABI self-description ------------------- ref: csrc/homura_rocm.h:589-610 */
/* ';'-separated offload architectures compiled in ("gfx950"). */
const char *hmr_built_archs(void);

typedef struct hmr_abi_info {
    uint32_t abi_info_size;
    uint32_t properties_size;
    uint32_t properties_align;
    uint32_t properties_offsets[5];
    int32_t status_values[5];
    int32_t name_len;
    int32_t arch_len;
    uint32_t desc_size;
    uint32_t desc_align;
    uint32_t desc_offsets[6];
    int32_t dtype_values[10];
    int32_t max_dims;
    uint32_t gemm_desc_size;
    uint32_t gemm_desc_align;
} hmr_abi_info;

/* Sizes, alignments, field offsets and enumerator values as this library was compiled. */
void hmr_abi_check(hmr_abi_info *out);

/* ---- test hooks ("not part of the supported interface") ----- ref: csrc/homura_rocm.h:612-666 */
/* Per calling thread: the next n stream creations / context creations after the probe /
 * property queries / data operations fail (data operations fail before queueing anything, as
 * out of memory when out_of_memory != 0, else as an invalid handle). */
void hmr_test_fail_stream_create(int32_t n);
void hmr_test_fail_after_probe(int32_t n);
void hmr_test_fail_properties(int32_t n);
void hmr_test_fail_data(int32_t n, int32_t out_of_memory);
/* The plan this library picks. The numbers describe THIS design and are not the reference's:
 *   group  = lanes that cooperate on one output (1, 64 = one wave, or the workgroup size),
 *   splits = workgroup slices the reduced range is cut into (>1 means a second pass),
 *   chunk  = reduced elements per slice. */
hmr_status hmr_test_reduce_plan(const hmr_tensor_desc *kept, const hmr_tensor_desc *red,
                                int64_t *group, int64_t *splits, int64_t *chunk);
/*   split = 0 (rows are never cut: one wave or one workgroup owns a row),
 *   group = lanes per row, cache = row elements a lane keeps in registers (0: the row is
 *   streamed twice instead). */
hmr_status hmr_test_softmax_plan(const hmr_tensor_desc *src_rows, int64_t n, int64_t src_stride,
                                 int32_t *split, int32_t *group, int32_t *cache);
/* ref :631-657  The second step of hmr_index_check alone: unless slot[0] (a logical position of `index`,
 * set by the caller) is UINT64_MAX, the value there goes to slot[1]. For positions far beyond what a
 * check could reach in a test (2^60 and more, in views with zero strides). */
hmr_status hmr_test_index_value(hmr_context_t ctx, const hmr_tensor_desc *index, uint64_t *slot);
int32_t hmr_test_live_streams(void);
hmr_status hmr_test_current_device(int32_t *device);
hmr_status hmr_test_set_current_device(int32_t device);
hmr_status hmr_test_fail(const char *message);

#ifdef __cplusplus
}
#endif

#endif /* HOMURA_ROCM_H */
