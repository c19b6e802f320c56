// hmr_binary_scalar, hmr_where, hmr_where_constant, hmr_fill
// (ref: csrc/homura_rocm.h:142, 217, 247-255; csrc/elementwise.hip:1035-1132, csrc/copy.hip:154-173).
#include "ew_common.hpp"

namespace hmr {
namespace {

template <class T>
uint64_t scalar_bits_of(double s) {
    using C = typename Comp<T>::C;
    C c = static_cast<C>(s);  // rounded to the computation type, as the CPU's C::of
    uint64_t bits = 0;
    __builtin_memcpy(&bits, &c, sizeof c);
    return bits;
}

// ---- fill of a contiguous, 16-byte aligned destination -------------------------------------------------
//
// Nothing is read: a thread stores kFillTiles tiles of 16 bytes, a workgroup's width apart; the first
// workgroup also writes the elements after the last whole tile. Other destinations go through the
// map kernels with the value as a constant operand.
constexpr int kFillTiles = 4;

template <class W>
__global__ void __launch_bounds__(kBlock) fill_kernel(char *out, int64_t n_tiles, int64_t n, W value) {
    constexpr int V = 16 / static_cast<int>(sizeof(W));
    W r[V];
#pragma unroll
    for (int i = 0; i < V; ++i) r[i] = value;
    const int64_t first = static_cast<int64_t>(blockIdx.x) * (kFillTiles * kBlock) + threadIdx.x;
#pragma unroll
    for (int u = 0; u < kFillTiles; ++u) {
        const int64_t t = first + static_cast<int64_t>(u) * kBlock;
        if (t < n_tiles) store_tile<W, V, false>(out + t * 16, r);
    }
    const int64_t done = n_tiles * V;
    if (blockIdx.x == 0 && done + threadIdx.x < n) reinterpret_cast<W *>(out)[done + threadIdx.x] = value;
}

template <class W>
bool launch_fill(const MapCall &c, uint64_t bits, hipStream_t stream) {
    constexpr int V = 16 / static_cast<int>(sizeof(W));
    const bool flat = c.ndim == 0 || (c.ndim == 1 && c.stride[0][0] == 1);
    if (!flat || reinterpret_cast<uintptr_t>(c.ptr[0]) % 16 != 0) return false;
    const int64_t n_tiles = c.n / V;
    const int64_t per_block = int64_t{kFillTiles} * kBlock;
    const int64_t blocks = n_tiles / per_block + 1;  // at least one, for the elements after the last tile
    if (blocks > (int64_t{1} << 22)) return false;
    W value;
    __builtin_memcpy(&value, &bits, sizeof(W));
    hipLaunchKernelGGL((fill_kernel<W>), dim3(static_cast<unsigned>(blocks)), dim3(kBlock), 0, stream, c.ptr[0], n_tiles, c.n,
                       value);
    return true;
}

}  // namespace
}  // namespace hmr

extern "C" {

hmr_status hmr_binary_scalar(hmr_context_t ctx, int32_t op, const hmr_tensor_desc *out, const hmr_tensor_desc *a,
                             double s, int32_t scalar_first) {
    return hmr::fenced([&] {
        if (op != HMR_BINARY_MUL && op != HMR_BINARY_DIV) {
            return hmr::fail(HMR_INVALID, "binary_scalar: only Mul and Div keep their scalar unrounded");
        }
        const int mode = op == HMR_BINARY_MUL ? 0 : (scalar_first ? 2 : 1);
        uint64_t bits = 0;
        bool is_float = hmr::with_float_type(a->dtype, [&](auto t) {
            bits = hmr::scalar_bits_of<typename decltype(t)::type>(s);
        });
        const hmr_tensor_desc *descs[3] = {out, a, nullptr};
        const uint64_t cbits[3] = {0, 0, bits};
        return hmr::run_map(ctx, "binary_scalar", 3, descs, cbits,
                            [&](const hmr::MapCall &call, hipStream_t stream) {
                                if (!is_float || out->dtype != a->dtype) return false;
                                return hmr::with_float_type(a->dtype, [&](auto t) {
                                    using T = typename decltype(t)::type;
                                    if (mode == 0) hmr::launch_map<hmr::ScalarBinary<0, T>>(call, stream);
                                    else if (mode == 1) hmr::launch_map<hmr::ScalarBinary<1, T>>(call, stream);
                                    else hmr::launch_map<hmr::ScalarBinary<2, T>>(call, stream);
                                });
                            });
    });
}

hmr_status hmr_where_constant(hmr_context_t ctx, const hmr_tensor_desc *out, const hmr_tensor_desc *cond,
                              const hmr_tensor_desc *x, uint64_t x_bits, const hmr_tensor_desc *y,
                              uint64_t y_bits) {
    return hmr::fenced([&] {
        const hmr_tensor_desc *descs[4] = {out, cond, x, y};
        const uint64_t cbits[4] = {0, 0, x_bits, y_bits};
        return hmr::run_map(ctx, "where", 4, descs, cbits, [&](const hmr::MapCall &call, hipStream_t stream) {
            if (cond->dtype != HMR_BOOL) return false;
            if ((x && x->dtype != out->dtype) || (y && y->dtype != out->dtype)) return false;
            return hmr::with_word(hmr::dtype_size(out->dtype), [&](auto w) {
                hmr::launch_map<hmr::Select<typename decltype(w)::type>>(call, stream);
            });
        });
    });
}

hmr_status hmr_where(hmr_context_t ctx, const hmr_tensor_desc *out, const hmr_tensor_desc *cond,
                     const hmr_tensor_desc *x, const hmr_tensor_desc *y) {
    if (x == nullptr || y == nullptr) return hmr::fail(HMR_INVALID, "where: a branch is missing");
    return hmr_where_constant(ctx, out, cond, x, 0, y, 0);
}

hmr_status hmr_fill(hmr_context_t ctx, const hmr_tensor_desc *dst, uint64_t bits) {
    return hmr::fenced([&] {
        const hmr_tensor_desc *descs[2] = {dst, nullptr};
        const uint64_t cbits[2] = {0, bits};
        return hmr::run_map(ctx, "fill", 2, descs, cbits, [&](const hmr::MapCall &call, hipStream_t stream) {
            return hmr::with_word(hmr::dtype_size(dst->dtype), [&](auto w) {
                using W = typename decltype(w)::type;
                if (!hmr::launch_fill<W>(call, bits, stream)) hmr::launch_map<hmr::Move<W>>(call, stream);
            });
        });
    });
}

}  // extern "C"
