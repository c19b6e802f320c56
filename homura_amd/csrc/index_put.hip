// hmr_index_positions, hmr_index_overwrite(+workspace), hmr_mask_workspace / hmr_mask_count / hmr_mask_coordinates
// (ref: csrc/homura_rocm.h:376-389, 415-426; the semantics are src/backend/cpu/misc.rs:104-203).
//
//   positions   one pass per indexed dimension of an advanced index: out = (first ? 0 : out) + wrapped
//               coordinate * stride, element by element over the broadcast shape.
//   overwrite   slice i of src goes to slice positions[i] of out and the last of repeated positions wins. Which i
//               is the last for a position does not depend on the order threads run in: a word per position
//               of out takes the maximum of i + 1 (an atomic maximum commutes), and then only the winners copy.
//   masks       the true elements are counted per tile of 4096, the tiles' counts are scanned by one workgroup
//               (the total is left where the host reads it), and a second pass over the mask writes the
//               coordinates of the k-th true element, k = the tile's offset + the rank inside the tile.
#include "mail.hpp"
#include "index.hpp"

namespace hmr {
namespace {

// ---- hmr_index_positions ------------------------------------------------------------------------------------

// stride[0] out, [1] the coordinates.
__global__ void __launch_bounds__(kBlock) positions_kernel(int64_t *out, const void *coord, int is64, Dims d, int64_t n, int64_t size,
                                                           int64_t stride, int first) {
    // Four positions per lane, a workgroup apart, every load before the first store; the outermost dimension
    // needs no division.
    constexpr int U = 4;
    for (int64_t base = static_cast<int64_t>(blockIdx.x) * (U * kBlock); base < n; base += static_cast<int64_t>(gridDim.x) * (U * kBlock)) {
        int64_t oo[U], v[U], before[U];
        bool valid[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int64_t wanted = base + static_cast<int64_t>(u) * kBlock + threadIdx.x;
            valid[u] = wanted < n;
            int64_t rest = valid[u] ? wanted : n - 1, co = 0;
            oo[u] = 0;
            for (int k = 0; k < d.ndim; ++k) {
                int64_t c = rest;
                if (k + 1 < d.ndim) {
                    const int64_t q = rest / d.size[k];
                    c = rest - q * d.size[k];
                    rest = q;
                }
                oo[u] += c * d.stride[0][k];
                co += c * d.stride[1][k];
            }
            v[u] = read_index(coord, is64, co);
            before[u] = first ? 0 : out[oo[u]];
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            if (v[u] < 0) v[u] += size;
            if (valid[u]) out[oo[u]] = before[u] + v[u] * stride;
        }
    }
}

// ---- hmr_index_overwrite ------------------------------------------------------------------------------------

__global__ void __launch_bounds__(kBlock) winners_clear_kernel(unsigned long long *winners, int64_t size) {
    for (int64_t j = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x; j < size; j += static_cast<int64_t>(gridDim.x) * kBlock) {
        winners[j] = 0;
    }
}

__global__ void __launch_bounds__(kBlock) winners_kernel(unsigned long long *winners, const void *positions, int is64,
                                                         int64_t position_stride, int64_t m) {
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x; i < m; i += static_cast<int64_t>(gridDim.x) * kBlock) {
        atomicMax(&winners[read_index(positions, is64, i * position_stride)], static_cast<unsigned long long>(i) + 1);
    }
}

// `d` holds the slice's dimensions (every dimension but the indexed one): stride[0] out, [1] src.
template <class W>
__global__ void __launch_bounds__(kBlock) overwrite_kernel(W *out, const W *src, const unsigned long long *winners, const void *positions,
                                                           int is64, int64_t position_stride, Dims d, int64_t m, int64_t slice,
                                                           int64_t out_step, int64_t src_step) {
    const int64_t n = m * slice;
    for (int64_t p = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x; p < n; p += static_cast<int64_t>(gridDim.x) * kBlock) {
        const int64_t i = p / slice;
        const int64_t j = read_index(positions, is64, i * position_stride);
        if (winners[j] != static_cast<unsigned long long>(i) + 1) continue;
        int64_t rest = p - i * slice, oo = 0, so = 0;
        for (int k = 0; k < d.ndim; ++k) {
            const int64_t q = rest / d.size[k];
            const int64_t c = rest - q * d.size[k];
            rest = q;
            oo += c * d.stride[0][k];
            so += c * d.stride[1][k];
        }
        out[oo + j * out_step] = src[so + i * src_step];
    }
}

// The same when a slice is one contiguous run of whole aligned 16-byte tiles in both operands.
template <class W>
__global__ void __launch_bounds__(kBlock) overwrite_tiles_kernel(W *out, const W *src, const unsigned long long *winners,
                                                                 const void *positions, int is64, int64_t position_stride, int64_t m,
                                                                 int64_t tiles, int64_t out_step, int64_t src_step) {
    constexpr int V = 16 / static_cast<int>(sizeof(W));
    const int64_t n = m * tiles;
    for (int64_t p = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x; p < n; p += static_cast<int64_t>(gridDim.x) * kBlock) {
        const int64_t i = p / tiles;
        const int64_t t = p - i * tiles;
        const int64_t j = read_index(positions, is64, i * position_stride);
        if (winners[j] != static_cast<unsigned long long>(i) + 1) continue;
        W r[V];
        load_tile<W, V, kStreamLoads>(reinterpret_cast<const char *>(src + i * src_step + t * V), r);
        store_tile<W, V, false>(reinterpret_cast<char *>(out + j * out_step + t * V), r);
    }
}

// ---- masks ----------------------------------------------------------------------------------------------------

constexpr int kMaskPerThread = 16;
constexpr int kMaskTile = kBlock * kMaskPerThread;

// The flags of the 16 elements first .. first + 15 (row-major positions) as a bit set; elements past n are 0.
// FLAT: the mask is contiguous from a 16-byte aligned address.
template <bool FLAT>
__device__ __forceinline__ uint32_t mask_bits(const uint8_t *mask, const Dims &d, int64_t first, int64_t n) {
    uint32_t bits = 0;
    if (first >= n) return 0;
    if constexpr (FLAT) {
        if (first + kMaskPerThread <= n) {
            const u32x4 v = *reinterpret_cast<const u32x4 *>(mask + first);
            const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
            for (int i = 0; i < kMaskPerThread; ++i) bits |= ((w[i / 4] >> (8 * (i % 4))) & 0xFFu) != 0 ? (1u << i) : 0u;
            return bits;
        }
        for (int i = 0; i < kMaskPerThread; ++i) {
            if (first + i < n && mask[first + i] != 0) bits |= 1u << i;
        }
        return bits;
    } else {
        // The coordinates of `first`, then a step at a time with carries.
        int64_t coord[kMaxIndexDims];
        int64_t rest = first, off = 0;
        for (int k = 0; k < d.ndim; ++k) {
            const int64_t q = rest / d.size[k];
            coord[k] = rest - q * d.size[k];
            off += coord[k] * d.stride[0][k];
            rest = q;
        }
        for (int i = 0; i < kMaskPerThread && first + i < n; ++i) {
            if (mask[off] != 0) bits |= 1u << i;
            for (int k = 0; k < d.ndim; ++k) {
                off += d.stride[0][k];
                if (++coord[k] < d.size[k]) break;
                off -= coord[k] * d.stride[0][k];
                coord[k] = 0;
            }
        }
        return bits;
    }
}

template <bool FLAT>
__global__ void __launch_bounds__(kBlock) mask_count_kernel(const uint8_t *mask, Dims d, int64_t n, int64_t tiles, uint64_t *counts) {
    __shared__ uint32_t lds[kBlock / 64];
    for (int64_t tile = blockIdx.x; tile < tiles; tile += gridDim.x) {
        uint32_t c = __popc(mask_bits<FLAT>(mask, d, tile * kMaskTile + static_cast<int64_t>(threadIdx.x) * kMaskPerThread, n));
#pragma unroll
        for (int m = 32; m >= 1; m >>= 1) c += static_cast<uint32_t>(__shfl_xor(static_cast<int>(c), m, 64));
        __syncthreads();  // lds is reused from tile to tile
        if ((threadIdx.x & 63) == 0) lds[threadIdx.x / 64] = c;
        __syncthreads();
        if (threadIdx.x == 0) {
            uint32_t total = 0;
            for (int w = 0; w < kBlock / 64; ++w) total += lds[w];
            counts[tile] = total;
        }
    }
}

// One workgroup: counts[0 .. tiles) become their exclusive prefix sums and counts[tiles] the total. A lane takes
// eight adjacent counts per step.
constexpr int kScanBlock = 1024;
constexpr int kScanPer = 8;
__global__ void __launch_bounds__(kScanBlock) mask_scan_kernel(uint64_t *counts, int64_t tiles, uint64_t *mailbox, uint64_t ticket) {
    __shared__ uint64_t lds[kScanBlock / 64];
    const int lane = threadIdx.x & 63, wave = threadIdx.x / 64;
    uint64_t carry = 0;
    for (int64_t base = 0; base < tiles; base += static_cast<int64_t>(kScanBlock) * kScanPer) {
        const int64_t first = base + static_cast<int64_t>(threadIdx.x) * kScanPer;
        uint64_t v[kScanPer];
        uint64_t sum = 0;
#pragma unroll
        for (int i = 0; i < kScanPer; ++i) {
            v[i] = first + i < tiles ? counts[first + i] : 0;
            sum += v[i];
        }
        uint64_t x = sum;
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
            const uint64_t lo = static_cast<uint32_t>(__shfl_up(static_cast<int>(x), off, 64));
            const uint64_t hi = static_cast<uint32_t>(__shfl_up(static_cast<int>(x >> 32), off, 64));
            if (lane >= off) x += (hi << 32) | lo;
        }
        if (lane == 63) lds[wave] = x;
        __syncthreads();
        uint64_t before = carry + x - sum, total = 0;
        for (int w = 0; w < kScanBlock / 64; ++w) {
            before += w < wave ? lds[w] : 0;
            total += lds[w];
        }
#pragma unroll
        for (int i = 0; i < kScanPer; ++i) {
            if (first + i < tiles) counts[first + i] = before;
            before += v[i];
        }
        carry += total;
        __syncthreads();
    }
    // The total also goes to the mailbox: the host reads it back at once, to size the result.
    if (threadIdx.x == 0) {
        counts[tiles] = carry;
        post(mailbox, ticket, carry, 0);
    }
}

// The same scan by many workgroups, for up to kSpreadTiles tiles: workgroup w owns 256 tiles, adds up every count
// before them (its lanes take every 256th, sixteen loads at a time; the counts of all earlier tiles are at most
// 512 KB, which the L2 serves) and scans its own. It reads `raw` and writes `offsets`, two arrays: a workgroup
// may still be reading counts that another has already replaced by offsets. One launch of some microseconds
// instead of two dependent passes of one workgroup.
constexpr int64_t kSpreadTiles = 65536;
__global__ void __launch_bounds__(kBlock) mask_scan_spread_kernel(const uint64_t *raw, uint64_t *offsets, int64_t tiles, uint64_t *mailbox,
                                                                  uint64_t ticket) {
    __shared__ uint64_t lds[kBlock / 64];
    const int lane = threadIdx.x & 63, wave = threadIdx.x / 64;
    const int64_t first = static_cast<int64_t>(blockIdx.x) * kBlock;
    auto fold = [&](uint64_t x) {  // the sum over the workgroup, in every lane
#pragma unroll
        for (int m = 32; m >= 1; m >>= 1) {
            const uint64_t lo = static_cast<uint32_t>(__shfl_xor(static_cast<int>(x), m, 64));
            const uint64_t hi = static_cast<uint32_t>(__shfl_xor(static_cast<int>(x >> 32), m, 64));
            x += (hi << 32) | lo;
        }
        __syncthreads();
        if (lane == 0) lds[wave] = x;
        __syncthreads();
        uint64_t total = 0;
        for (int w = 0; w < kBlock / 64; ++w) total += lds[w];
        return total;
    };
    constexpr int kAhead = 16;  // loads in flight per lane: the last workgroup of 65 536 tiles reads 255 counts a lane
    uint64_t sum = 0;
    int64_t j = threadIdx.x;
    for (; j + (kAhead - 1) * kBlock < first; j += kAhead * kBlock) {
        uint64_t got[kAhead];
#pragma unroll
        for (int u = 0; u < kAhead; ++u) got[u] = raw[j + u * kBlock];
#pragma unroll
        for (int u = 0; u < kAhead; ++u) sum += got[u];
    }
    for (; j < first; j += kBlock) sum += raw[j];
    const uint64_t before = fold(sum);
    // The workgroup's own 256 counts: an inclusive scan along the lanes, then across the waves.
    const int64_t mine = first + threadIdx.x;
    const uint64_t v = mine < tiles ? raw[mine] : 0;
    uint64_t x = v;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
        const uint64_t lo = static_cast<uint32_t>(__shfl_up(static_cast<int>(x), off, 64));
        const uint64_t hi = static_cast<uint32_t>(__shfl_up(static_cast<int>(x >> 32), off, 64));
        if (lane >= off) x += (hi << 32) | lo;
    }
    __syncthreads();
    if (lane == 63) lds[wave] = x;
    __syncthreads();
    uint64_t ahead = before;
    for (int w = 0; w < wave; ++w) ahead += lds[w];
    if (mine < tiles) offsets[mine] = ahead + x - v;
    if (mine == tiles - 1) {
        const uint64_t total = ahead + x;
        offsets[tiles] = total;
        post(mailbox, ticket, total, 0);
    }
}

// Division by the mask's sizes (innermost first) for positions below 2^31.
struct MaskDivs {
    FastDiv d[kMaxIndexDims];
};

// out[dim][k] at out + dim * out_row + k * out_col. The true elements of a tile are first compacted into LDS
// (their places inside the tile, in order), then lane j takes the tile's j-th, j + 256-th, ... of them: the
// stores of a wave fill whole lines of each row of out. SMALL: n < 2^31, coordinates by multiplication.
// STREAM: nontemporal stores (rows that are contiguous only).
template <bool FLAT, bool SMALL, bool STREAM>
__global__ void __launch_bounds__(kBlock) mask_write_kernel(const uint8_t *mask, Dims d, MaskDivs divs, int64_t n, int64_t tiles,
                                                            const uint64_t *offsets, int64_t *out, int64_t count, int64_t out_row,
                                                            int64_t out_col) {
    __shared__ uint32_t lds[kBlock / 64];
    __shared__ uint16_t place[kMaskTile];
    const int lane = threadIdx.x & 63, wave = threadIdx.x / 64;
    for (int64_t tile = blockIdx.x; tile < tiles; tile += gridDim.x) {
        const int64_t first = tile * kMaskTile + static_cast<int64_t>(threadIdx.x) * kMaskPerThread;
        const uint32_t bits = mask_bits<FLAT>(mask, d, first, n);
        const uint32_t c = __popc(bits);
        uint32_t x = c;
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
            const uint32_t y = static_cast<uint32_t>(__shfl_up(static_cast<int>(x), off, 64));
            if (lane >= off) x += y;
        }
        __syncthreads();  // lds and place are reused from tile to tile
        if (lane == 63) lds[wave] = x;
        __syncthreads();
        uint32_t rank = x - c;
        for (int w = 0; w < wave; ++w) rank += lds[w];
        for (uint32_t rest_bits = bits; rest_bits != 0; rest_bits &= rest_bits - 1) {
            place[rank++] = static_cast<uint16_t>(threadIdx.x * kMaskPerThread + (__ffs(rest_bits) - 1));
        }
        __syncthreads();
        const int64_t k0 = static_cast<int64_t>(offsets[tile]);
        const uint32_t in_tile = static_cast<uint32_t>(offsets[tile + 1] - offsets[tile]);
        for (uint32_t j = threadIdx.x; j < in_tile; j += kBlock) {
            const int64_t k = k0 + j;
            if (k >= count) break;
            const int64_t linear = tile * kMaskTile + place[j];
            int64_t *po = out + k * out_col;
            if constexpr (SMALL) {
                if (out_col == 1) break;  // rows that are contiguous are written below, a row at a time
                uint32_t rest = static_cast<uint32_t>(linear);
                for (int dd = 0; dd < d.ndim - 1; ++dd) {
                    const uint32_t q = divide(rest, divs.d[dd]);
                    po[(d.ndim - 1 - dd) * out_row] = rest - q * divs.d[dd].div;
                    rest = q;
                }
                if (d.ndim > 0) po[0] = rest;
            } else {
                int64_t rest = linear;
                for (int dd = 0; dd < d.ndim - 1; ++dd) {
                    const int64_t q = rest / d.size[dd];
                    po[(d.ndim - 1 - dd) * out_row] = rest - q * d.size[dd];
                    rest = q;
                }
                if (d.ndim > 0) po[0] = rest;
            }
        }
        if constexpr (SMALL) {
            if (out_col == 1) {
                // A row of the output at a time, the lanes shifted so that each wave's 64 stores begin on a 128-byte
                // line of that row: whole lines then leave the compute unit in one piece, whatever the tile's offset.
                for (int row = 0; row < d.ndim; ++row) {
                    int64_t *prow = out + row * out_row;
                    const int shift = static_cast<int>((reinterpret_cast<uintptr_t>(prow + k0) >> 3) & 15u);
                    for (int j = static_cast<int>(threadIdx.x) - shift; j < static_cast<int>(in_tile); j += kBlock) {
                        if (j < 0) continue;
                        const int64_t k = k0 + j;
                        if (k >= count) break;
                        uint32_t rest = static_cast<uint32_t>(tile * kMaskTile + place[j]);
                        for (int dd = 0; dd < d.ndim - 1 - row; ++dd) rest = divide(rest, divs.d[dd]);
                        if (row > 0) rest -= divide(rest, divs.d[d.ndim - 1 - row]) * divs.d[d.ndim - 1 - row].div;
                        if constexpr (STREAM) __builtin_nontemporal_store(static_cast<int64_t>(rest), prow + k);
                        else prow[k] = rest;
                    }
                }
            }
        }
    }
}

int64_t mask_tiles(int64_t n) { return (n + kMaskTile - 1) / kMaskTile; }

bool mask_is_flat(const hmr_tensor_desc &mask) {
    int64_t stride = 1;
    for (int k = mask.ndim - 1; k >= 0; --k) {
        if (mask.sizes[k] != 1 && mask.strides[k] != stride) return false;
        stride *= mask.sizes[k];
    }
    return reinterpret_cast<uintptr_t>(first_of(mask)) % 16 == 0;
}

}  // namespace
}  // namespace hmr

using hmr::fail;
using hmr::fenced;

extern "C" {

hmr_status hmr_index_positions(hmr_context_t ctx, const hmr_tensor_desc *out, const hmr_tensor_desc *coord, int64_t size, int64_t stride,
                               int32_t first) {
    return fenced([&] {
        int64_t n = 0, m = 0;
        if (hmr_status s = hmr::check_desc(*out, n)) return s;
        if (hmr_status s = hmr::check_desc(*coord, m)) return s;
        if (out->dtype != HMR_I64) return fail(HMR_INVALID, "index_positions: the positions are I64");
        if (!hmr::is_index_dtype(coord->dtype)) return fail(HMR_INVALID, "index_positions: unsupported dtype");
        if (hmr_status s = hmr::check_same_sizes(*out, *coord, -1)) return s;
        if (n == 0) return HMR_OK;
        const hmr_tensor_desc *const ops[3] = {out, coord, nullptr};
        const hmr::Dims d = hmr::dims_of(*out, ops, -1);
        return hmr::queue_on(ctx, "index_positions", [&](hipStream_t stream) {
            hipLaunchKernelGGL(hmr::positions_kernel, dim3(hmr::grid_of((n + 3) / 4)), dim3(hmr::kBlock), 0, stream,
                               reinterpret_cast<int64_t *>(hmr::first_of(*out)), static_cast<const void *>(hmr::first_of(*coord)),
                               coord->dtype == HMR_I64 ? 1 : 0, d, n, size, stride, first);
            return true;
        });
    });
}

hmr_status hmr_index_overwrite_workspace(int64_t size, int64_t *bytes) {
    return fenced([&] {
        if (size < 0) return fail(HMR_INVALID, "index_overwrite_workspace: negative size");
        *bytes = size * 8;
        return HMR_OK;
    });
}

hmr_status hmr_index_overwrite(hmr_context_t ctx, const hmr_tensor_desc *out, const hmr_tensor_desc *src,
                               const hmr_tensor_desc *positions, int32_t dim, void *workspace, int64_t workspace_bytes) {
    return fenced([&] {
        int64_t n = 0, total = 0, m = 0;
        if (hmr_status s = hmr::check_desc(*out, n)) return s;
        if (hmr_status s = hmr::check_desc(*src, total)) return s;
        if (hmr_status s = hmr::check_desc(*positions, m)) return s;
        if (dim < 0 || dim >= out->ndim) return fail(HMR_INVALID, "index_overwrite: the dimension is out of range");
        if (hmr_status s = hmr::check_same_sizes(*out, *src, dim)) return s;
        if (positions->ndim > 1 || m != src->sizes[dim]) return fail(HMR_INVALID, "index_overwrite: the positions don't match the source");
        if (!hmr::is_index_dtype(positions->dtype)) return fail(HMR_INVALID, "index_overwrite: unsupported dtype");
        if (src->dtype != out->dtype) return fail(HMR_INVALID, "index_overwrite: unsupported dtype");
        if (total == 0) return HMR_OK;
        const int64_t size = out->sizes[dim];
        if (workspace == nullptr || workspace_bytes < size * 8) return fail(HMR_INVALID, "index_overwrite: the workspace is too small");
        hmr_tensor_desc so = *out, ss = *src;
        int kept = 0;
        for (int k = 0; k < out->ndim; ++k) {
            if (k == dim) continue;
            so.sizes[kept] = out->sizes[k];
            so.strides[kept] = out->strides[k];
            ss.strides[kept] = src->strides[k];
            ++kept;
        }
        so.ndim = kept;
        const hmr_tensor_desc *const ops[3] = {&so, &ss, nullptr};
        const hmr::Dims d = hmr::dims_of(so, ops, -1);
        const int64_t slice = total / m;
        const int elem = hmr::dtype_size(out->dtype);
        const int vec = 16 / elem;
        const int is64 = positions->dtype == HMR_I64 ? 1 : 0;
        const int64_t position_stride = positions->ndim == 1 ? positions->strides[0] : 0;
        const void *pos = hmr::first_of(*positions);
        unsigned long long *winners = static_cast<unsigned long long *>(workspace);
        const bool tiles = (d.ndim == 0 || (d.ndim == 1 && d.stride[0][0] == 1 && d.stride[1][0] == 1)) && slice % vec == 0 &&
                           reinterpret_cast<uintptr_t>(hmr::first_of(*out)) % 16 == 0 &&
                           reinterpret_cast<uintptr_t>(hmr::first_of(*src)) % 16 == 0 && out->strides[dim] % vec == 0 &&
                           src->strides[dim] % vec == 0;
        return hmr::queue_on(ctx, "index_overwrite", [&](hipStream_t stream) {
            hipLaunchKernelGGL(hmr::winners_clear_kernel, dim3(hmr::grid_of(size)), dim3(hmr::kBlock), 0, stream, winners, size);
            hipLaunchKernelGGL(hmr::winners_kernel, dim3(hmr::grid_of(m)), dim3(hmr::kBlock), 0, stream, winners, pos, is64, position_stride,
                               m);
            return hmr::with_word(elem, [&](auto w) {
                using W = typename decltype(w)::type;
                W *po = reinterpret_cast<W *>(hmr::first_of(*out));
                const W *ps = reinterpret_cast<const W *>(hmr::first_of(*src));
                if (tiles) {
                    hipLaunchKernelGGL((hmr::overwrite_tiles_kernel<W>), dim3(hmr::grid_of(m * (slice / vec))), dim3(hmr::kBlock), 0, stream,
                                       po, ps, static_cast<const unsigned long long *>(winners), pos, is64, position_stride, m,
                                       slice / vec, out->strides[dim], src->strides[dim]);
                } else {
                    hipLaunchKernelGGL((hmr::overwrite_kernel<W>), dim3(hmr::grid_of(total)), dim3(hmr::kBlock), 0, stream, po, ps,
                                       static_cast<const unsigned long long *>(winners), pos, is64, position_stride, d, m, slice,
                                       out->strides[dim], src->strides[dim]);
                }
            });
        });
    });
}

hmr_status hmr_mask_workspace(int64_t n, int64_t *bytes, int64_t *total_word) {
    return fenced([&] {
        if (n < 0) return fail(HMR_INVALID, "mask_workspace: negative size");
        const int64_t tiles = hmr::mask_tiles(n);
        // The tiles' offsets and the total, then the tiles' raw counts where the spread scan wants them apart.
        *bytes = (tiles + 1 + (tiles <= hmr::kSpreadTiles ? tiles : 0)) * 8;
        *total_word = tiles;
        return HMR_OK;
    });
}

hmr_status hmr_mask_count(hmr_context_t ctx, const hmr_tensor_desc *mask, void *workspace, int64_t workspace_bytes) {
    return fenced([&] {
        int64_t n = 0;
        if (hmr_status s = hmr::check_desc(*mask, n)) return s;
        if (mask->dtype != HMR_BOOL) return fail(HMR_INVALID, "mask_count: the mask is BOOL");
        const int64_t tiles = hmr::mask_tiles(n);
        const bool spread = tiles > 0 && tiles <= hmr::kSpreadTiles;
        if (workspace == nullptr || workspace_bytes < (tiles + 1 + (spread ? tiles : 0)) * 8) {
            return fail(HMR_INVALID, "mask_count: the workspace is too small");
        }
        const hmr_tensor_desc *const ops[3] = {mask, nullptr, nullptr};
        const hmr::Dims d = hmr::dims_of(*mask, ops, -1);
        const uint8_t *base = reinterpret_cast<const uint8_t *>(hmr::first_of(*mask));
        uint64_t *offsets = static_cast<uint64_t *>(workspace);
        uint64_t *counts = spread ? offsets + tiles + 1 : offsets;
        const bool flat = hmr::mask_is_flat(*mask);
        const int64_t cap = int64_t{1} << 20;
        if (ctx == nullptr) return fail(HMR_INVALID, "mask_count: null context");
        uint64_t *mailbox = static_cast<uint64_t *>(ctx->mailbox);
        const uint64_t ticket = ++ctx->mail_ticket;
        const hmr_status queued = hmr::queue_on(ctx, "mask_count", [&](hipStream_t stream) {
            if (tiles > 0) {
                const dim3 grid(static_cast<unsigned>(tiles < cap ? tiles : cap));
                if (flat) hipLaunchKernelGGL((hmr::mask_count_kernel<true>), grid, dim3(hmr::kBlock), 0, stream, base, d, n, tiles, counts);
                else hipLaunchKernelGGL((hmr::mask_count_kernel<false>), grid, dim3(hmr::kBlock), 0, stream, base, d, n, tiles, counts);
            }
            if (spread) {
                hipLaunchKernelGGL(hmr::mask_scan_spread_kernel, dim3(static_cast<unsigned>((tiles + hmr::kBlock - 1) / hmr::kBlock)),
                                   dim3(hmr::kBlock), 0, stream, counts, offsets, tiles, mailbox, ticket);
            } else {
                hipLaunchKernelGGL(hmr::mask_scan_kernel, dim3(1), dim3(hmr::kScanBlock), 0, stream, counts, tiles, mailbox, ticket);
            }
            return true;
        });
        // The total is in the mailbox as well once the scan has run: a read-back of that word takes it from there.
        if (queued == HMR_OK) ctx->mail_src = offsets + tiles;
        return queued;
    });
}

hmr_status hmr_mask_coordinates(hmr_context_t ctx, const hmr_tensor_desc *mask, void *workspace, int64_t workspace_bytes,
                                const hmr_tensor_desc *out) {
    return fenced([&] {
        int64_t n = 0, total = 0;
        if (hmr_status s = hmr::check_desc(*mask, n)) return s;
        if (hmr_status s = hmr::check_desc(*out, total)) return s;
        if (mask->dtype != HMR_BOOL) return fail(HMR_INVALID, "mask_coordinates: the mask is BOOL");
        if (out->dtype != HMR_I64 || out->ndim != 2 || out->sizes[0] != mask->ndim) {
            return fail(HMR_INVALID, "mask_coordinates: the output is I64, the mask's rank x the number of true elements");
        }
        const int64_t tiles = hmr::mask_tiles(n);
        if (workspace == nullptr || workspace_bytes < (tiles + 1) * 8) return fail(HMR_INVALID, "mask_coordinates: the workspace is too small");
        if (total == 0 || tiles == 0) return HMR_OK;
        const hmr_tensor_desc *const ops[3] = {mask, nullptr, nullptr};
        const hmr::Dims d = hmr::dims_of(*mask, ops, -1);
        const uint8_t *base = reinterpret_cast<const uint8_t *>(hmr::first_of(*mask));
        const uint64_t *offsets = static_cast<const uint64_t *>(workspace);
        int64_t *po = reinterpret_cast<int64_t *>(hmr::first_of(*out));
        const bool flat = hmr::mask_is_flat(*mask);
        const bool small = n < (int64_t{1} << 31);
        hmr::MaskDivs divs{};
        for (int k = 0; small && k < d.ndim; ++k) divs.d[k] = hmr::make_fastdiv(static_cast<uint32_t>(d.size[k]));
        const int64_t cap = int64_t{1} << 20;
        // Coordinates that the memory-side cache (256 MB) cannot hold for their reader go past the caches: with the
        // stores of a wave on whole lines, 644 MB of them took 165 us that way and 192 us through the caches, and
        // the picks that follow 322 MB of positions 30 us less.
        const int past_caches = total * 8 >= (int64_t{256} << 20) ? 1 : 0;
        return hmr::queue_on(ctx, "mask_coordinates", [&](hipStream_t stream) {
            const dim3 grid(static_cast<unsigned>(tiles < cap ? tiles : cap));
            auto run = [&](auto flat_tag, auto small_tag) {
                constexpr bool kFlat = decltype(flat_tag)::value, kSmall = decltype(small_tag)::value;
                if constexpr (kSmall) {
                    if (past_caches) {
                        hipLaunchKernelGGL((hmr::mask_write_kernel<kFlat, true, true>), grid, dim3(hmr::kBlock), 0, stream, base, d, divs, n,
                                           tiles, offsets, po, out->sizes[1], out->strides[0], out->strides[1]);
                        return;
                    }
                }
                hipLaunchKernelGGL((hmr::mask_write_kernel<kFlat, kSmall, false>), grid, dim3(hmr::kBlock), 0, stream, base, d, divs, n,
                                   tiles, offsets, po, out->sizes[1], out->strides[0], out->strides[1]);
            };
            if (flat && small) run(std::true_type{}, std::true_type{});
            else if (flat) run(std::true_type{}, std::false_type{});
            else if (small) run(std::false_type{}, std::true_type{});
            else run(std::false_type{}, std::false_type{});
            return true;
        });
    });
}

}  // extern "C"
