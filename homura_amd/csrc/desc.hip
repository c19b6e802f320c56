// Validation and dimension merging of operand descriptions (host code).
// Checks follow ref: csrc/kernel.hpp:62-121; merging follows the rule of the caller's
// merge_dims (ref: src/backend/rocm/copy.rs:33-57), re-applied here so that a caller that did
// not merge still reaches the fast kernels.
#include "map.hpp"

namespace hmr {

hmr_status check_desc(const hmr_tensor_desc &d, int64_t &n, bool negative_strides) {
    if (d.dtype < HMR_BOOL || d.dtype > HMR_F64) return fail(HMR_INVALID, "invalid dtype " + std::to_string(d.dtype));
    if (d.ndim < 0 || d.ndim > HMR_MAX_DIMS) {
        return fail(HMR_INVALID, "invalid number of dimensions " + std::to_string(d.ndim));
    }
    n = 1;
    bool empty = false, wraps = false;
    for (int k = 0; k < d.ndim; ++k) {
        if (d.sizes[k] < 0) return fail(HMR_INVALID, "negative size");
        if (d.strides[k] < 0 && !negative_strides) return fail(HMR_INVALID, "negative stride");
        empty = empty || d.sizes[k] == 0;
        wraps = __builtin_mul_overflow(n, d.sizes[k], &n) || wraps;
    }
    if (empty) n = 0;  // whatever the other sizes are
    else if (wraps) return fail(HMR_INVALID, "the number of elements does not fit 64 bits");
    return HMR_OK;
}

hmr_status prepare_map(MapCall &c, int count, const hmr_tensor_desc *const *descs, const uint64_t *bits,
                       bool negative_inputs) {
    const hmr_tensor_desc &out = *descs[0];
    c.nops = count;
    if (hmr_status s = check_desc(out, c.n)) return s;
    for (int k = 0; k < count; ++k) {
        c.is_const[k] = descs[k] == nullptr;
        c.cbits[k] = bits ? bits[k] : 0;
        c.ptr[k] = nullptr;
        c.elem_size[k] = 0;
        if (c.is_const[k]) continue;
        const hmr_tensor_desc &d = *descs[k];
        if (k > 0) {
            int64_t m = 0;
            if (hmr_status s = check_desc(d, m, negative_inputs)) return s;
            bool same = d.ndim == out.ndim;
            for (int j = 0; same && j < out.ndim; ++j) same = d.sizes[j] == out.sizes[j];
            if (!same) return fail(HMR_INVALID, "kernel operands have different sizes");
        }
        c.elem_size[k] = dtype_size(d.dtype);
        c.ptr[k] = static_cast<char *>(d.data) + d.offset * c.elem_size[k];
    }
    c.ndim = 0;
    if (c.n == 0) return HMR_OK;
    for (int i = 0; i < out.ndim; ++i) {
        int64_t size = out.sizes[i];
        if (size == 1) continue;
        bool joins = c.ndim > 0;
        for (int k = 0; joins && k < count; ++k) {
            if (c.is_const[k]) continue;
            int64_t prod = 0;
            joins = !__builtin_mul_overflow(descs[k]->strides[i], size, &prod) && prod == c.stride[k][c.ndim - 1];
        }
        if (joins) {
            c.size[c.ndim - 1] *= size;
            for (int k = 0; k < count; ++k) c.stride[k][c.ndim - 1] = c.is_const[k] ? 0 : descs[k]->strides[i];
        } else {
            c.size[c.ndim] = size;
            for (int k = 0; k < count; ++k) c.stride[k][c.ndim] = c.is_const[k] ? 0 : descs[k]->strides[i];
            ++c.ndim;
        }
    }
    return HMR_OK;
}

}  // namespace hmr
