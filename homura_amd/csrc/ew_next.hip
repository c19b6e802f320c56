// hmr_fused, hmr_triangle, hmr_flip
// (ref: csrc/homura_rocm.h:195-263; csrc/elementwise.hip:334-371, 554-575, 1048-1175).
#include "ew_common.hpp"

namespace hmr {
namespace {

template <class T>
uint64_t coefficient_bits(double v) {
    using C = typename Comp<T>::C;
    C c = static_cast<C>(v);  // the caller passes a value of the computation type; this is exact
    uint64_t bits = 0;
    __builtin_memcpy(&bits, &c, sizeof c);
    return bits;
}

// ---- triangle ---------------------------------------------------------------------------------------
//
// The matrix dimensions are the last two of the descriptions; the ones before are batch
// dimensions. A thread owns V adjacent columns of one row (V elements = 16 bytes when both rows are
// contiguous and aligned, else 1) and writes src or zeros; a tile that lies wholly outside the
// kept triangle is not read at all.
struct TriangleArgs {
    char *out;
    const char *src;
    int64_t n_tiles;       // tiles over (batch, row, column tile)
    uint32_t rows, cols, tiles_per_row;
    FastDiv tiles_div, rows_div;
    int32_t nbatch;        // merged batch dimensions, innermost first
    FastDiv batch_div[HMR_MAX_DIMS];
    int64_t batch_stride[2][HMR_MAX_DIMS];
    int64_t row_stride[2], col_stride[2];
    int64_t diagonal;
    int32_t upper;
};

template <class W, int V>
__global__ void __launch_bounds__(kBlock) triangle_kernel(TriangleArgs a) {
    for (int64_t t = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x; t < a.n_tiles;
         t += static_cast<int64_t>(gridDim.x) * kBlock) {
        // t = (batch * rows + row) * tiles_per_row + tile; every factor fits 31 bits (checked on the host).
        const uint32_t line = divide(static_cast<uint32_t>(t), a.tiles_div);
        const uint32_t tile = static_cast<uint32_t>(t) - line * a.tiles_per_row;
        uint32_t batch = divide(line, a.rows_div);
        const uint32_t row = line - batch * a.rows;
        int64_t oo = static_cast<int64_t>(row) * a.row_stride[0], so = static_cast<int64_t>(row) * a.row_stride[1];
        for (int d = 0; d < a.nbatch; ++d) {
            const uint32_t q = divide(batch, a.batch_div[d]);
            const uint32_t idx = batch - q * a.batch_div[d].div;
            batch = q;
            oo += idx * a.batch_stride[0][d];
            so += idx * a.batch_stride[1][d];
        }
        const int64_t c0 = static_cast<int64_t>(tile) * V;
        // keep(c) = upper ? c - row >= diagonal : c - row <= diagonal: a range of columns.
        const int64_t edge = static_cast<int64_t>(row) + a.diagonal;  // upper: keep c >= edge; lower: keep c <= edge
        W *po = reinterpret_cast<W *>(a.out) + oo + c0 * a.col_stride[0];
        const W *ps = reinterpret_cast<const W *>(a.src) + so + c0 * a.col_stride[1];
        if constexpr (V > 1) {
            const bool none = a.upper ? c0 + V - 1 < edge : c0 > edge;
            W r[V] = {};
            if (!none) {
                load_tile<W, V, false>(reinterpret_cast<const char *>(ps), r);
#pragma unroll
                for (int i = 0; i < V; ++i) {
                    const bool keep = a.upper ? c0 + i >= edge : c0 + i <= edge;
                    r[i] = keep ? r[i] : W{};
                }
            }
            store_tile<W, V, false>(reinterpret_cast<char *>(po), r);
        } else {
            const bool keep = a.upper ? c0 >= edge : c0 <= edge;
            *po = keep ? *ps : W{};
        }
    }
}

template <class W>
void launch_triangle(const hmr_tensor_desc &out, const hmr_tensor_desc &src, int64_t diagonal, int upper,
                     hipStream_t stream) {
    const int nd = out.ndim;
    TriangleArgs a{};
    a.out = static_cast<char *>(out.data) + out.offset * static_cast<int64_t>(sizeof(W));
    a.src = static_cast<const char *>(src.data) + src.offset * static_cast<int64_t>(sizeof(W));
    a.rows = static_cast<uint32_t>(out.sizes[nd - 2]);
    a.cols = static_cast<uint32_t>(out.sizes[nd - 1]);
    a.row_stride[0] = out.strides[nd - 2];
    a.row_stride[1] = src.strides[nd - 2];
    a.col_stride[0] = out.strides[nd - 1];
    a.col_stride[1] = src.strides[nd - 1];
    // Row and column indices are below 2^31, so a diagonal beyond that keeps everything or nothing:
    // clamping it keeps `row + diagonal` inside int64.
    constexpr int64_t kFar = int64_t{1} << 40;
    a.diagonal = diagonal < -kFar ? -kFar : (diagonal > kFar ? kFar : diagonal);
    a.upper = upper;
    a.nbatch = 0;
    int64_t batches = 1;
    for (int d = nd - 3; d >= 0; --d) {
        if (out.sizes[d] == 1) continue;
        a.batch_div[a.nbatch] = make_fastdiv(static_cast<uint32_t>(out.sizes[d]));
        a.batch_stride[0][a.nbatch] = out.strides[d];
        a.batch_stride[1][a.nbatch] = src.strides[d];
        ++a.nbatch;
        batches *= out.sizes[d];
    }
    constexpr int kVec = 16 / static_cast<int>(sizeof(W));
    bool vec = a.col_stride[0] == 1 && a.col_stride[1] == 1 && a.cols % kVec == 0 &&
               reinterpret_cast<uintptr_t>(a.out) % 16 == 0 && reinterpret_cast<uintptr_t>(a.src) % 16 == 0 &&
               (a.row_stride[0] * sizeof(W)) % 16 == 0 && (a.row_stride[1] * sizeof(W)) % 16 == 0;
    for (int d = 0; vec && d < a.nbatch; ++d) {
        vec = (a.batch_stride[0][d] * sizeof(W)) % 16 == 0 && (a.batch_stride[1][d] * sizeof(W)) % 16 == 0;
    }
    const int v = vec ? kVec : 1;
    a.tiles_per_row = a.cols / v;
    a.tiles_div = make_fastdiv(a.tiles_per_row);
    a.rows_div = make_fastdiv(a.rows);
    a.n_tiles = batches * a.rows * a.tiles_per_row;
    const unsigned grid = grid_for(a.n_tiles, kBlock);
    if (vec) hipLaunchKernelGGL((triangle_kernel<W, kVec>), dim3(grid), dim3(kBlock), 0, stream, a);
    else hipLaunchKernelGGL((triangle_kernel<W, 1>), dim3(grid), dim3(kBlock), 0, stream, a);
}

}  // namespace
}  // namespace hmr

extern "C" {

hmr_status hmr_fused(hmr_context_t ctx, int32_t op, const hmr_tensor_desc *out, const hmr_tensor_desc *a,
                     const hmr_tensor_desc *b, const hmr_tensor_desc *c, double coefficient, int32_t small) {
    return hmr::guarded([&] {
        if (op < HMR_FUSED_SCALED_ADD || op > HMR_FUSED_ADDCDIV) return hmr::fail(HMR_INVALID, "fused: unknown step");
        const bool three = op >= HMR_FUSED_ADDCMUL;
        if (three != (c != nullptr)) {
            return hmr::fail(HMR_INVALID, three ? "fused: the step needs three operands" : "fused: the step takes two operands");
        }
        uint64_t bits = 0;
        const bool is_float = hmr::with_float_type(out->dtype, [&](auto t) {
            bits = hmr::coefficient_bits<typename decltype(t)::type>(coefficient);
        });
        const hmr_tensor_desc *descs[4] = {out, a, b, c};
        const uint64_t cbits[4] = {bits, 0, 0, 0};
        return hmr::run_map(ctx, "fused", three ? 4 : 3, descs, cbits, [&](const hmr::MapCall &call, hipStream_t stream) {
            if (!is_float || a->dtype != out->dtype || b->dtype != out->dtype || (c && c->dtype != out->dtype)) return false;
            return hmr::with_float_type(out->dtype, [&](auto t) {
                using T = typename decltype(t)::type;
                switch (op) {
                    case HMR_FUSED_SCALED_ADD: hmr::launch_map<hmr::FusedStep<HMR_FUSED_SCALED_ADD, T, false>>(call, stream); break;
                    case HMR_FUSED_LERP:
                        if (small) hmr::launch_map<hmr::FusedStep<HMR_FUSED_LERP, T, true>>(call, stream);
                        else hmr::launch_map<hmr::FusedStep<HMR_FUSED_LERP, T, false>>(call, stream);
                        break;
                    case HMR_FUSED_ADDCMUL: hmr::launch_map<hmr::FusedStep<HMR_FUSED_ADDCMUL, T, false>>(call, stream); break;
                    default: hmr::launch_map<hmr::FusedStep<HMR_FUSED_ADDCDIV, T, false>>(call, stream); break;
                }
            });
        });
    });
}

hmr_status hmr_triangle(hmr_context_t ctx, const hmr_tensor_desc *out, const hmr_tensor_desc *src, int64_t diagonal,
                        int32_t upper) {
    return hmr::guarded([&] {
        int64_t n = 0, m = 0;
        if (hmr_status s = hmr::check_desc(*out, n)) return s;
        if (hmr_status s = hmr::check_desc(*src, m)) return s;
        bool same = src->ndim == out->ndim;
        for (int j = 0; same && j < out->ndim; ++j) same = src->sizes[j] == out->sizes[j];
        if (!same) return hmr::fail(HMR_INVALID, "kernel operands have different sizes");
        if (out->ndim < 2) return hmr::fail(HMR_INVALID, "triangle needs two dimensions");
        if (n == 0) return HMR_OK;
        if (n >= (int64_t{1} << 31)) return hmr::fail(HMR_INVALID, "triangle: more than 2^31 - 1 elements");
        return hmr::launch_on(ctx, "triangle", [&](hipStream_t stream) {
            if (src->dtype != out->dtype) return false;
            return hmr::with_word(hmr::dtype_size(out->dtype), [&](auto w) {
                hmr::launch_triangle<typename decltype(w)::type>(*out, *src, diagonal, upper != 0, stream);
            });
        });
    });
}

hmr_status hmr_flip(hmr_context_t ctx, const hmr_tensor_desc *out, const hmr_tensor_desc *src) {
    return hmr::guarded([&] {
        const hmr_tensor_desc *descs[2] = {out, src};
        return hmr::run_map(
            ctx, "flip", 2, descs, nullptr,
            [&](const hmr::MapCall &call, hipStream_t stream) {
                if (src->dtype != out->dtype) return false;
                return hmr::with_word(hmr::dtype_size(out->dtype), [&](auto w) {
                    hmr::launch_map<hmr::Move<typename decltype(w)::type>>(call, stream);
                });
            },
            [](const hmr::MapCall &) { return HMR_OK; }, /*negative_inputs=*/true);
    });
}

}  // extern "C"
