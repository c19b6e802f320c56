// What the indexing kernels share: the walk over the dimensions of a call and the reading of I32 / I64 positions.
#pragma once

#include "ew_common.hpp"

namespace hmr {

constexpr int kMaxIndexDims = HMR_MAX_DIMS;

// The dimensions shared by the operands of a call, innermost first, with up to three stride sets.
struct Dims {
    int32_t ndim;
    int32_t at;  // the indexed dimension, counted from the innermost
    int64_t size[kMaxIndexDims];
    int64_t stride[3][kMaxIndexDims];
};

__device__ __forceinline__ int64_t read_index(const void *base, int is64, int64_t offset) {
    return is64 ? static_cast<const int64_t *>(base)[offset] : static_cast<int64_t>(static_cast<const int32_t *>(base)[offset]);
}

inline unsigned grid_of(int64_t threads) {
    const int64_t want = (threads + kBlock - 1) / kBlock;
    const int64_t cap = int64_t{1} << 20;
    return static_cast<unsigned>(want < 1 ? 1 : (want < cap ? want : cap));
}

inline bool is_index_dtype(int dtype) { return dtype == HMR_I32 || dtype == HMR_I64; }

// The dimensions of `shape_of` (sizes) with the strides of up to three operands, innermost first.
// `dim` (counted from the outermost, as in the descriptions) becomes `at`.
inline Dims dims_of(const hmr_tensor_desc &shape_of, const hmr_tensor_desc *const (&ops)[3], int dim) {
    Dims d{};
    d.ndim = shape_of.ndim;
    d.at = dim < 0 ? -1 : shape_of.ndim - 1 - dim;
    for (int k = 0; k < shape_of.ndim; ++k) {
        const int from = shape_of.ndim - 1 - k;
        d.size[k] = shape_of.sizes[from];
        for (int o = 0; o < 3; ++o) d.stride[o][k] = ops[o] ? ops[o]->strides[from] : 0;
    }
    return d;
}

// The same walk without the dimensions of one element (their coordinate is always 0), `at` kept whatever its size:
// the element kernels divide once per dimension and element.
inline Dims squeezed(const Dims &d) {
    Dims s{};
    s.at = -1;
    for (int k = 0; k < d.ndim; ++k) {
        if (d.size[k] == 1 && k != d.at) continue;
        if (k == d.at) s.at = s.ndim;
        s.size[s.ndim] = d.size[k];
        for (int o = 0; o < 3; ++o) s.stride[o][s.ndim] = d.stride[o][k];
        ++s.ndim;
    }
    return s;
}

inline char *first_of(const hmr_tensor_desc &d) { return static_cast<char *>(d.data) + d.offset * dtype_size(d.dtype); }

// The largest offset (in elements) a walk over `sizes` with `strides` reaches.
inline int64_t reach_of(const hmr_tensor_desc &d) {
    int64_t reach = 0;
    for (int k = 0; k < d.ndim; ++k) reach += (d.sizes[k] - 1) * d.strides[k];
    return reach;
}

inline hmr_status check_same_sizes(const hmr_tensor_desc &a, const hmr_tensor_desc &b, int except) {
    bool same = a.ndim == b.ndim;
    for (int k = 0; same && k < a.ndim; ++k) same = k == except || a.sizes[k] == b.sizes[k];
    return same ? HMR_OK : fail(HMR_INVALID, "kernel operands have different sizes");
}

}  // namespace hmr
