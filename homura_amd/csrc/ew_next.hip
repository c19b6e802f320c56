// hmr_fused, hmr_addr, hmr_triangle, hmr_flip
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

// ---- triangle and flip: rows of 16-byte tiles ---------------------------------------------------
//
// Both write a tensor whose innermost dimension is contiguous from a source whose innermost stride
// is 1 (triangle, flip of outer dimensions) or -1 (flip of the innermost one). The innermost two
// dimensions are (row, column); the ones before are batch dimensions, whose strides (like the
// source's row stride) may be negative for flip. A thread owns kTilesPerThread tiles of V adjacent
// columns (16 bytes) a workgroup's width apart and issues all its loads before it uses any.
//   triangle   a tile wholly outside the kept triangle reads the row's tile at the diagonal
//              instead (which a neighbour reads anyway) and writes zeros;
//   reversed   the tile is read from the mirrored position and its elements are swapped around.
// Operands that aren't made of aligned whole tiles take the element kernels.
constexpr int kTilesPerThread = 4;
enum TileMode { kTriangle = 0, kCopy = 1, kReversed = 2 };

struct TileArgs {
    char *out;
    const char *src;       // element (0, .., 0) of the source: with a reversed row, its last in memory
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

// Offsets (in elements) of the row that tile `t` lies in, its row index and its column tile.
__device__ __forceinline__ void locate(const TileArgs &a, uint32_t t, int64_t &oo, int64_t &so, uint32_t &row,
                                       uint32_t &tile) {
    // t = (batch * rows + row) * tiles_per_row + tile; every factor fits 31 bits (checked on the host).
    const uint32_t line = divide(t, a.tiles_div);
    tile = t - line * a.tiles_per_row;
    uint32_t batch = divide(line, a.rows_div);
    row = line - batch * a.rows;
    oo = static_cast<int64_t>(row) * a.row_stride[0];
    so = static_cast<int64_t>(row) * a.row_stride[1];
    for (int d = 0; d < a.nbatch; ++d) {
        const uint32_t q = divide(batch, a.batch_div[d]);
        const int64_t idx = batch - q * a.batch_div[d].div;
        batch = q;
        oo += idx * a.batch_stride[0][d];
        so += idx * a.batch_stride[1][d];
    }
}

template <class W, int MODE>
__global__ void __launch_bounds__(kBlock) tiles_kernel(TileArgs a) {
    constexpr int V = 16 / static_cast<int>(sizeof(W));
    constexpr int U = kTilesPerThread;
    const int64_t first = static_cast<int64_t>(blockIdx.x) * (U * kBlock) + threadIdx.x;
    W r[U][V];
    int64_t oo[U], edge[U], c0[U];
    bool valid[U], none[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
        const int64_t t = first + static_cast<int64_t>(u) * kBlock;
        valid[u] = t < a.n_tiles;
        int64_t so;
        uint32_t row, tile;
        locate(a, static_cast<uint32_t>(valid[u] ? t : a.n_tiles - 1), oo[u], so, row, tile);
        c0[u] = static_cast<int64_t>(tile) * V;
        oo[u] += c0[u];
        int64_t from = so + c0[u];
        none[u] = false;
        if constexpr (MODE == kTriangle) {
            // keep(c) = upper ? c - row >= diagonal : c - row <= diagonal: columns from `edge` on, or up to it.
            edge[u] = static_cast<int64_t>(row) + a.diagonal;
            none[u] = a.upper ? c0[u] + V - 1 < edge[u] : c0[u] > edge[u];
            int64_t at = edge[u] < 0 ? 0 : (edge[u] >= a.cols ? a.cols - 1 : edge[u]);
            at -= at % V;
            from = so + (none[u] ? at : c0[u]);
        } else if constexpr (MODE == kReversed) {
            from = so - c0[u] - (V - 1);
        }
        if constexpr (MODE == kTriangle) {
            // A wave whose tiles all lie outside the triangle reads nothing (a wave-uniform branch).
            if (__builtin_amdgcn_ballot_w64(!none[u]) != 0) {
                load_tile<W, V, kStreamLoads>(a.src + from * static_cast<int64_t>(sizeof(W)), r[u]);
            } else {
#pragma unroll
                for (int i = 0; i < V; ++i) r[u][i] = W{};
            }
        } else {
            load_tile<W, V, kStreamLoads>(a.src + from * static_cast<int64_t>(sizeof(W)), r[u]);
        }
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int u = 0; u < U; ++u) {
        W w[V];
#pragma unroll
        for (int i = 0; i < V; ++i) {
            if constexpr (MODE == kTriangle) {
                const bool keep = !none[u] && (a.upper ? c0[u] + i >= edge[u] : c0[u] + i <= edge[u]);
                w[i] = keep ? r[u][i] : W{};
            } else if constexpr (MODE == kReversed) {
                w[i] = r[u][V - 1 - i];
            } else {
                w[i] = r[u][i];
            }
        }
        if (valid[u]) store_tile<W, V, false>(a.out + oo[u] * static_cast<int64_t>(sizeof(W)), w);
    }
}

// One element per thread: triangles of operands that aren't made of aligned whole tiles.
template <class W>
__global__ void __launch_bounds__(kBlock) triangle_elements_kernel(TileArgs a) {
    for (int64_t t = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x; t < a.n_tiles;
         t += static_cast<int64_t>(gridDim.x) * kBlock) {
        int64_t oo, so;
        uint32_t row, col;
        locate(a, static_cast<uint32_t>(t), oo, so, row, col);
        const int64_t edge = static_cast<int64_t>(row) + a.diagonal;
        const bool keep = a.upper ? col >= edge : col <= edge;
        const W *ps = reinterpret_cast<const W *>(a.src) + so + col * a.col_stride[1];
        reinterpret_cast<W *>(a.out)[oo + col * a.col_stride[0]] = keep ? *ps : W{};
    }
}

// Whether both operands are rows of whole aligned tiles; `reversed`: the source's rows run backwards.
template <class W>
bool tiles_apply(const TileArgs &a, bool reversed) {
    constexpr int kVec = 16 / static_cast<int>(sizeof(W));
    if (a.col_stride[0] != 1 || a.col_stride[1] != (reversed ? -1 : 1) || a.cols % kVec != 0) return false;
    // The first tile a row's column 0 belongs to starts V - 1 elements before it when the row is reversed.
    const uintptr_t src = reinterpret_cast<uintptr_t>(a.src) - (reversed ? (kVec - 1) * sizeof(W) : 0);
    if (reinterpret_cast<uintptr_t>(a.out) % 16 != 0 || src % 16 != 0) return false;
    auto whole = [](int64_t stride) { return stride % kVec == 0; };
    if (a.rows > 1 && (!whole(a.row_stride[0]) || !whole(a.row_stride[1]))) return false;
    for (int d = 0; d < a.nbatch; ++d) {
        if (!whole(a.batch_stride[0][d]) || !whole(a.batch_stride[1][d])) return false;
    }
    return true;
}

// Takes the sizes and strides (outermost first) of `nd` >= 1 dimensions of both operands.
inline TileArgs tile_args(void *out, const void *src, int nd, const int64_t *sizes, const int64_t *out_strides,
                          const int64_t *src_strides) {
    TileArgs a{};
    a.out = static_cast<char *>(out);
    a.src = static_cast<const char *>(src);
    a.rows = nd >= 2 ? static_cast<uint32_t>(sizes[nd - 2]) : 1;
    a.cols = static_cast<uint32_t>(sizes[nd - 1]);
    a.row_stride[0] = nd >= 2 ? out_strides[nd - 2] : 0;
    a.row_stride[1] = nd >= 2 ? src_strides[nd - 2] : 0;
    a.col_stride[0] = out_strides[nd - 1];
    a.col_stride[1] = src_strides[nd - 1];
    a.nbatch = 0;
    for (int d = nd - 3; d >= 0; --d) {
        if (sizes[d] == 1) continue;
        a.batch_div[a.nbatch] = make_fastdiv(static_cast<uint32_t>(sizes[d]));
        a.batch_stride[0][a.nbatch] = out_strides[d];
        a.batch_stride[1][a.nbatch] = src_strides[d];
        ++a.nbatch;
    }
    a.rows_div = make_fastdiv(a.rows);
    return a;
}

inline void set_tiles(TileArgs &a, int64_t n, int per_tile) {
    a.tiles_per_row = a.cols / per_tile;
    a.tiles_div = make_fastdiv(a.tiles_per_row);
    a.n_tiles = n / per_tile;
}

template <class W, int MODE>
void launch_tiles(TileArgs &a, int64_t n, hipStream_t stream) {
    set_tiles(a, n, 16 / static_cast<int>(sizeof(W)));
    const unsigned grid = grid_for(a.n_tiles, int64_t{kTilesPerThread} * kBlock);
    hipLaunchKernelGGL((tiles_kernel<W, MODE>), dim3(grid), dim3(kBlock), 0, stream, a);
}

template <class W>
void launch_triangle(const hmr_tensor_desc &out, const hmr_tensor_desc &src, int64_t n, int64_t diagonal, int upper,
                     hipStream_t stream) {
    TileArgs a = tile_args(static_cast<char *>(out.data) + out.offset * static_cast<int64_t>(sizeof(W)),
                           static_cast<const char *>(src.data) + src.offset * static_cast<int64_t>(sizeof(W)), out.ndim,
                           out.sizes, out.strides, src.strides);
    // Row and column indices are below 2^31, so a diagonal beyond that keeps everything or nothing:
    // clamping it keeps `row + diagonal` inside int64.
    constexpr int64_t kFar = int64_t{1} << 40;
    a.diagonal = diagonal < -kFar ? -kFar : (diagonal > kFar ? kFar : diagonal);
    a.upper = upper;
    if (tiles_apply<W>(a, false)) {
        launch_tiles<W, kTriangle>(a, n, stream);
    } else {
        set_tiles(a, n, 1);
        hipLaunchKernelGGL((triangle_elements_kernel<W>), dim3(grid_for(n, kBlock)), dim3(kBlock), 0, stream, a);
    }
}

// A flip whose merged operands are rows of whole tiles; false leaves it to the element kernels.
template <class W>
bool launch_flip_tiles(const MapCall &c, hipStream_t stream) {
    if (c.ndim < 1 || c.n >= (int64_t{1} << 31)) return false;
    TileArgs a = tile_args(c.ptr[0], c.ptr[1], c.ndim, c.size, c.stride[0], c.stride[1]);
    const bool reversed = a.col_stride[1] == -1;
    if (!tiles_apply<W>(a, reversed)) return false;
    if (reversed) launch_tiles<W, kReversed>(a, c.n, stream);
    else launch_tiles<W, kCopy>(a, c.n, stream);
    return true;
}

}  // namespace
}  // namespace hmr

extern "C" {

hmr_status hmr_fused(hmr_context_t ctx, int32_t op, const hmr_tensor_desc *out, const hmr_tensor_desc *a,
                     const hmr_tensor_desc *b, const hmr_tensor_desc *c, double coefficient, int32_t small) {
    return hmr::fenced([&] {
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

hmr_status hmr_addr(hmr_context_t ctx, const hmr_tensor_desc *out, const hmr_tensor_desc *v1, const hmr_tensor_desc *v2,
                    const hmr_tensor_desc *input, double alpha, double beta, int64_t alpha_int, int64_t beta_int) {
    return hmr::fenced([&] {
        const bool is_float = out->dtype >= HMR_F16 && out->dtype <= HMR_F64;
        const bool is_bool = out->dtype == HMR_BOOL;
        // The coefficients as the kernels take them: bits of the computation type, i64, or 0 / 1.
        uint64_t cbits[4] = {0, 0, 0, 0};
        bool reads = false;
        if (is_float) {
            hmr::with_float_type(out->dtype, [&](auto t) {
                using T = typename decltype(t)::type;
                cbits[0] = hmr::coefficient_bits<T>(alpha);
                cbits[1] = hmr::coefficient_bits<T>(beta);
            });
            reads = beta != 0.0;  // a NaN beta reads the input, as the CPU's `beta != 0` does
        } else {
            cbits[0] = is_bool ? static_cast<uint64_t>(alpha_int != 0) : static_cast<uint64_t>(alpha_int);
            cbits[1] = is_bool ? static_cast<uint64_t>(beta_int != 0) : static_cast<uint64_t>(beta_int);
            reads = beta_int != 0;
        }
        if (out->ndim != 2) return hmr::fail(HMR_INVALID, "addr: the output must have two dimensions");
        if (reads && input == nullptr) return hmr::fail(HMR_INVALID, "addr: beta isn't zero but there is no input");
        const hmr_tensor_desc *descs[4] = {out, v1, v2, reads ? input : nullptr};
        return hmr::run_map(ctx, "addr", reads ? 4 : 3, descs, cbits, [&](const hmr::MapCall &call, hipStream_t stream) {
            if (v1->dtype != out->dtype || v2->dtype != out->dtype || (reads && input->dtype != out->dtype)) return false;
            if (is_bool) {
                if (reads) hmr::launch_map<hmr::AddrBool<true>>(call, stream);
                else hmr::launch_map<hmr::AddrBool<false>>(call, stream);
                return true;
            }
            auto launch = [&](auto t) {
                using T = typename decltype(t)::type;
                if constexpr (hmr::Conv<T>::kind == hmr::Kind::Float) {
                    if (reads) hmr::launch_map<hmr::AddrFloat<T, true>>(call, stream);
                    else hmr::launch_map<hmr::AddrFloat<T, false>>(call, stream);
                } else {
                    if (reads) hmr::launch_map<hmr::AddrInt<T, true>>(call, stream);
                    else hmr::launch_map<hmr::AddrInt<T, false>>(call, stream);
                }
            };
            return hmr::with_int_type(out->dtype, launch) || hmr::with_float_type(out->dtype, launch);
        });
    });
}

hmr_status hmr_triangle(hmr_context_t ctx, const hmr_tensor_desc *out, const hmr_tensor_desc *src, int64_t diagonal,
                        int32_t upper) {
    return hmr::fenced([&] {
        int64_t n = 0, m = 0;
        if (hmr_status s = hmr::check_desc(*out, n)) return s;
        if (hmr_status s = hmr::check_desc(*src, m)) return s;
        bool same = src->ndim == out->ndim;
        for (int j = 0; same && j < out->ndim; ++j) same = src->sizes[j] == out->sizes[j];
        if (!same) return hmr::fail(HMR_INVALID, "kernel operands have different sizes");
        if (out->ndim < 2) return hmr::fail(HMR_INVALID, "triangle needs two dimensions");
        if (n == 0) return HMR_OK;
        if (n >= (int64_t{1} << 31)) return hmr::fail(HMR_INVALID, "triangle: more than 2^31 - 1 elements");
        return hmr::queue_on(ctx, "triangle", [&](hipStream_t stream) {
            if (src->dtype != out->dtype) return false;
            return hmr::with_word(hmr::dtype_size(out->dtype), [&](auto w) {
                hmr::launch_triangle<typename decltype(w)::type>(*out, *src, n, diagonal, upper != 0, stream);
            });
        });
    });
}

hmr_status hmr_flip(hmr_context_t ctx, const hmr_tensor_desc *out, const hmr_tensor_desc *src) {
    return hmr::fenced([&] {
        const hmr_tensor_desc *descs[2] = {out, src};
        return hmr::run_map(
            ctx, "flip", 2, descs, nullptr,
            [&](const hmr::MapCall &call, hipStream_t stream) {
                if (src->dtype != out->dtype) return false;
                return hmr::with_word(hmr::dtype_size(out->dtype), [&](auto w) {
                    using W = typename decltype(w)::type;
                    if (!hmr::launch_flip_tiles<W>(call, stream)) hmr::launch_map<hmr::Move<W>>(call, stream);
                });
            },
            [](const hmr::MapCall &) { return HMR_OK; }, /*negative_inputs=*/true);
    });
}

}  // extern "C"
