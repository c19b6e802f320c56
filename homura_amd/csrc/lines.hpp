// What the entry points that work on "lines" of a tensor share (softmax rows, cumulative products): the check of
// the two descriptions of the lines and their merge into one walk per operand.
#pragma once

#include "reduce.hpp"

namespace hmr {

// Merges the line dimensions with respect to both operands, innermost first; returns the number of lines.
inline int64_t walk_pair(const hmr_tensor_desc &out_rows, const hmr_tensor_desc &src_rows, Walk &wo, Walk &ws) {
    // Merge the row dimensions with respect to both operands, innermost first.
    int64_t size[HMR_MAX_DIMS], so[HMR_MAX_DIMS], ss[HMR_MAX_DIMS];
    int n = 0;
    int64_t count = 1;
    for (int i = 0; i < src_rows.ndim; ++i) count *= src_rows.sizes[i];
    wo.ndim = ws.ndim = 0;
    if (count == 0) return 0;
    for (int i = 0; i < src_rows.ndim; ++i) {
        int64_t sz = src_rows.sizes[i];
        if (sz == 1) continue;
        int64_t p1 = 0, p2 = 0;
        if (n > 0 && !__builtin_mul_overflow(out_rows.strides[i], sz, &p1) && p1 == so[n - 1] &&
            !__builtin_mul_overflow(src_rows.strides[i], sz, &p2) && p2 == ss[n - 1]) {
            size[n - 1] *= sz;
            so[n - 1] = out_rows.strides[i];
            ss[n - 1] = src_rows.strides[i];
        } else {
            size[n] = sz;
            so[n] = out_rows.strides[i];
            ss[n] = src_rows.strides[i];
            ++n;
        }
    }
    wo.ndim = ws.ndim = n;
    for (int i = 0; i < n; ++i) {
        wo.size[i] = ws.size[i] = size[n - 1 - i];
        wo.stride[i] = so[n - 1 - i];
        ws.stride[i] = ss[n - 1 - i];
    }
    return count;
}

inline hmr_status check_rows(const hmr_tensor_desc &out_rows, const hmr_tensor_desc &src_rows, int64_t n, int64_t so,
                      int64_t si, int64_t &nrows) {
    int64_t m = 0;
    if (hmr_status s = check_desc(out_rows, nrows)) return s;
    if (hmr_status s = check_desc(src_rows, m)) return s;
    bool same = out_rows.ndim == src_rows.ndim;
    for (int j = 0; same && j < out_rows.ndim; ++j) same = out_rows.sizes[j] == src_rows.sizes[j];
    if (!same) return fail(HMR_INVALID, "kernel operands have different sizes");
    if (n < 0 || so < 0 || si < 0) return fail(HMR_INVALID, "invalid row length or stride");
    return HMR_OK;
}

}  // namespace hmr
