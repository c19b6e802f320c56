// Unary operations on 16-bit floats by table.
//
// A 16-bit element has 65 536 patterns, so any unary operation on f16 or bf16 is a 128 KiB table
// from input pattern to output pattern. The table is filled once per context, operation and dtype
// by applying the operation's own functor (the one the direct kernels use) to every pattern, so a
// looked-up result has the direct kernel's bits by construction. The lookup kernel keeps the table
// in LDS (128 KiB of the 160 KiB a CU has: one 1024-lane workgroup per CU) and streams the tensor
// past it: 16-byte loads and (write-through) stores, eight LDS reads per chunk, no arithmetic. What makes this worth
// it is the cost of the exact operations - erf goes through an f64 series of up to forty terms per
// element - against a kernel that runs at the speed of memory whatever the operation is.
#pragma once

#include "map.hpp"

namespace hmr {

constexpr int kTableBlock = 1024;
// Chunks a lane has in flight per pass: four over views (a pass is then whole 4 KiB runs of the output, see
// TableSplit), one over a contiguous tensor, where a 134 MB -> 134 MB lookup from and to HBM took 47.8 us with four,
// 47.2 with two and 45.8 with one (50.2 with eight).
constexpr int kTableTiles = 4;
constexpr int kTableTilesFlat = 1;
constexpr int kTableEntries = 1 << 16;
constexpr size_t kTableBytes = size_t{kTableEntries} * 2;
// Below this the direct kernel runs. Measured on bf16, per call with the host's 4 us included: the lookup takes
// 4.2 to 4.8 us from 2^15 to 2^21 elements whatever the operation, the direct kernel 6.5 to 8.5 us for exp, silu,
// sigmoid, sin, erf and gelu, 11 us for log, 21 us for log_sigmoid and 37 to 39 us for tanh and gelu_tanh (a lane
// of the direct kernel works through 32 elements one after the other, and the host library's tanhf is some two
// hundred dependent instructions with branches).
constexpr int64_t kTableMinElements = int64_t{1} << 15;

// table[pattern] = F(pattern) for every 16-bit pattern.
template <class F>
__global__ void __launch_bounds__(kBlock) table_fill_kernel(uint16_t *table) {
    using T = typename F::In0;
    static_assert(sizeof(T) == 2 && sizeof(typename F::Out) == 2, "16-bit operations only");
    const uint32_t i = blockIdx.x * kBlock + threadIdx.x;
    if (i < kTableEntries) {
        T x;
        x.bits = static_cast<uint16_t>(i);
        table[i] = F{}(x).bits;
    }
}

// How the walk over the outer dimensions splits for a launch of the table kernel whose passes keep step with
// them: a pass of a workgroup covers `rows_per_pass` whole rows, `low_rows` (the product of the first
// `low_dims` outer dimensions) is a multiple of that, and the rows between a workgroup's passes (the grid
// times `rows_per_pass`) are a multiple of `low_rows`. Then the coordinates of a lane's chunks along the low
// dimensions are the same in every pass, and those along the others are the same for the whole workgroup.
struct TableSplit {
    int32_t low_dims;       // 0: no such split, every chunk walks all dimensions
    uint32_t rows_per_pass;
    FastDiv low_rows;
};

// out = table[src] over the rows layout (see map_rows_kernel): FLAT, or an innermost dimension that
// is a multiple of the 8-element chunk below up to 5 outer dimensions. SPLIT (see TableSplit): the offsets of
// a lane's chunks are found once, before the passes, and a pass adds the workgroup's offset, which scalar
// instructions compute. The workgroup is the only one on its CU (the table fills LDS), so what its waves
// spend on offsets is time without loads in flight: on a bf16 [8, 2048, 32, 128] view permuted to
// [8, 32, 2048, 128] a walk over four dimensions per chunk took 46.3 us, none takes 42.3.
template <bool FLAT, bool SPLIT = false>
__global__ void __launch_bounds__(kTableBlock) map_table_kernel(RowsArgs<2> a, const uint16_t *table, TableSplit split) {
    constexpr int V = 8, U = FLAT ? kTableTilesFlat : kTableTiles;
    static_assert(!(FLAT && SPLIT), "the split is one of outer dimensions");
    __shared__ uint16_t lut[kTableEntries];
    {
        const u32x4 *from = reinterpret_cast<const u32x4 *>(table);
        u32x4 *to = reinterpret_cast<u32x4 *>(lut);
#pragma unroll
        for (int i = 0; i < static_cast<int>(kTableBytes / 16 / kTableBlock); ++i) {
            to[i * kTableBlock + threadIdx.x] = from[i * kTableBlock + threadIdx.x];
        }
    }
    __syncthreads();
    using Off = std::conditional_t<FLAT, int64_t, uint32_t>;
    const OutStores stores(a.ptr[0], a.out32 != 0);
    const int64_t tiles = (a.n + V - 1) / V;
    const int64_t whole = a.n / V;
    auto offsets = [&](int64_t t, Off &out_off, Off &src_off) {
        if constexpr (FLAT) {
            out_off = src_off = t * V;
        } else {
            const uint32_t e32 = static_cast<uint32_t>(t * V);
            uint32_t row = divide(e32, a.inner_div);
            const uint32_t col = e32 - row * a.inner;
            out_off = src_off = col;
            for (int d = 0; d < a.nouter; ++d) {
                const uint32_t q = divide(row, a.div[d]);
                const uint32_t idx = row - q * a.div[d].div;
                row = q;
                out_off += idx * static_cast<uint32_t>(a.ostride[0][d]);
                src_off += idx * static_cast<uint32_t>(a.ostride[1][d]);
            }
        }
    };
    auto lookup = [&](const u32x4 &raw) {
        u32x4 res;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const uint32_t w = raw[j];
            res[j] = static_cast<uint32_t>(lut[w & 0xFFFFu]) | (static_cast<uint32_t>(lut[w >> 16]) << 16);
        }
        return res;
    };
    if constexpr (SPLIT) {
        // The low part: the rows of this workgroup's passes start at the same place inside `low_rows`.
        const uint32_t first = blockIdx.x * split.rows_per_pass;
        const uint32_t first_low = first - divide(first, split.low_rows) * split.low_rows.div;
        uint32_t low_out[U], low_src[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const uint32_t e32 = static_cast<uint32_t>(u * kTableBlock + threadIdx.x) * V;
            const uint32_t r = divide(e32, a.inner_div);
            uint32_t row = first_low + r;
            low_out[u] = low_src[u] = e32 - r * a.inner;
            for (int d = 0; d < split.low_dims; ++d) {
                const uint32_t q = divide(row, a.div[d]);
                const uint32_t idx = row - q * a.div[d].div;
                row = q;
                low_out[u] += idx * static_cast<uint32_t>(a.ostride[0][d]);
                low_src[u] += idx * static_cast<uint32_t>(a.ostride[1][d]);
            }
        }
        const uint32_t passes = static_cast<uint32_t>(tiles / (U * kTableBlock));  // whole ones only
        for (uint32_t pass = blockIdx.x; pass < passes; pass += gridDim.x) {
            uint32_t row = divide(pass * split.rows_per_pass, split.low_rows);
            uint32_t high_out = 0, high_src = 0;
            for (int d = split.low_dims; d < a.nouter; ++d) {
                const uint32_t q = divide(row, a.div[d]);
                const uint32_t idx = row - q * a.div[d].div;
                row = q;
                high_out += idx * static_cast<uint32_t>(a.ostride[0][d]);
                high_src += idx * static_cast<uint32_t>(a.ostride[1][d]);
            }
            const char *src = a.ptr[1] + static_cast<int64_t>(high_src) * 2;
            u32x4 raw[U];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const u32x4 *q = reinterpret_cast<const u32x4 *>(src + static_cast<int64_t>(low_src[u]) * 2);
                if constexpr (kStreamLoads) raw[u] = __builtin_nontemporal_load(q);
                else raw[u] = *q;
            }
#pragma unroll
            for (int u = 0; u < U; ++u) {
                stores.put16((static_cast<int64_t>(high_out) + static_cast<int64_t>(low_out[u])) * 2, lookup(raw[u]));
            }
        }
        return;
    }
    for (int64_t base = static_cast<int64_t>(blockIdx.x) * (U * kTableBlock); base < tiles;
         base += static_cast<int64_t>(gridDim.x) * (U * kTableBlock)) {
        const int64_t t0 = base + threadIdx.x;
        if (base + U * kTableBlock <= whole) {
            u32x4 raw[U];
            Off oo[U];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                Off so;
                offsets(t0 + static_cast<int64_t>(u) * kTableBlock, oo[u], so);
                const u32x4 *q = reinterpret_cast<const u32x4 *>(a.ptr[1] + static_cast<int64_t>(so) * 2);
                if constexpr (kStreamLoads) raw[u] = __builtin_nontemporal_load(q);
                else raw[u] = *q;
            }
#pragma unroll
            for (int u = 0; u < U; ++u) {
                stores.put16(static_cast<int64_t>(oo[u]) * 2, lookup(raw[u]));
            }
        } else {
            for (int u = 0; u < U; ++u) {
                const int64_t t = t0 + static_cast<int64_t>(u) * kTableBlock;
                if (t >= tiles) break;
                const int64_t rem = a.n - t * V;
                const int valid = rem >= V ? V : static_cast<int>(rem);
                Off oo, so;
                offsets(t, oo, so);
                const uint16_t *ps = reinterpret_cast<const uint16_t *>(a.ptr[1] + static_cast<int64_t>(so) * 2);
                uint16_t *po = reinterpret_cast<uint16_t *>(a.ptr[0] + static_cast<int64_t>(oo) * 2);
                for (int i = 0; i < valid; ++i) po[i] = lut[ps[i]];
            }
        }
    }
}

// Whether `c` (a unary call on 16-bit elements) can take the table kernel: a rows layout with the
// source read as plain chunks, and enough elements to pay for filling 256 LDS copies of the table.
template <class F>
bool table_applies(const MapCall &c) {
    if (c.n < kTableMinElements || c.is_const[1]) return false;
    const int variant = resolve_variant<F>(c);
    if (variant > 1) return false;
    return c.ndim > 0 && c.stride[1][c.ndim - 1] == 1;
}

template <class F>
void launch_table_fill(uint16_t *table, hipStream_t stream) {
    hipLaunchKernelGGL((table_fill_kernel<F>), dim3(kTableEntries / kBlock), dim3(kBlock), 0, stream, table);
}

// The split of a launch of `blocks` workgroups over the layout `a` (see TableSplit), low_dims 0 if there is none.
inline TableSplit table_split(const RowsArgs<2> &a, int64_t tiles, int64_t blocks) {
    TableSplit none{0, 0, make_fastdiv(1)};
    constexpr int64_t kPass = kTableTiles * kTableBlock;  // chunks of a pass
    if (a.nouter < 1 || a.inner % 8 != 0 || tiles % kPass != 0) return none;
    const int64_t per_row = a.inner / 8;
    if (kPass % per_row != 0) return none;
    const int64_t rows_per_pass = kPass / per_row;
    int64_t low_rows = 1;
    for (int d = 0; d < a.nouter; ++d) {
        low_rows *= a.div[d].div;
        if (low_rows >= (int64_t{1} << 31)) return none;
        if (low_rows % rows_per_pass == 0 && (blocks * rows_per_pass) % low_rows == 0) {
            return TableSplit{d + 1, static_cast<uint32_t>(rows_per_pass), make_fastdiv(static_cast<uint32_t>(low_rows))};
        }
    }
    return none;
}

template <class F>
void launch_table(const MapCall &c, uint16_t *table, hipStream_t stream) {
    const int variant = resolve_variant<F>(c);
    RowsArgs<2> a = rows_args<F>(c, variant);
    const int64_t tiles = (c.n + 7) / 8;
    const int64_t per_pass = int64_t{variant == 0 ? kTableTilesFlat : kTableTiles} * kTableBlock;
    int64_t blocks = (tiles + per_pass - 1) / per_pass;
    if (blocks > c.compute_units) blocks = c.compute_units;  // one resident workgroup per CU, each loops
    const dim3 grid(static_cast<unsigned>(blocks)), block(kTableBlock);
    if (variant == 0) {
        hipLaunchKernelGGL((map_table_kernel<true>), grid, block, 0, stream, a, table, TableSplit{});
        return;
    }
    const TableSplit split = table_split(a, tiles, blocks);
    if (split.low_dims > 0) {
        hipLaunchKernelGGL((map_table_kernel<false, true>), grid, block, 0, stream, a, table, split);
    } else {
        hipLaunchKernelGGL((map_table_kernel<false>), grid, block, 0, stream, a, table, split);
    }
}

}  // namespace hmr
