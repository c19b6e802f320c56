// Unary operations on 16-bit floats by table.
//
// A 16-bit element has 65 536 patterns, so any unary operation on f16 or bf16 is a 128 KiB table
// from input pattern to output pattern. The table is filled once per context, operation and dtype
// by applying the operation's own functor (the one the direct kernels use) to every pattern, so a
// looked-up result has the direct kernel's bits by construction. The lookup kernel keeps the table
// in LDS (128 KiB of the 160 KiB a CU has: one 1024-lane workgroup per CU) and streams the tensor
// past it: 16-byte loads and stores, eight LDS reads per chunk, no arithmetic. What makes this worth
// it is the cost of the exact operations - erf goes through an f64 series of up to forty terms per
// element - against a kernel that runs at the speed of memory whatever the operation is.
#pragma once

#include "map.hpp"

namespace hmr {

constexpr int kTableBlock = 1024;
constexpr int kTableEntries = 1 << 16;
constexpr size_t kTableBytes = size_t{kTableEntries} * 2;
constexpr int64_t kTableMinElements = int64_t{1} << 20;  // below this the direct kernel is as fast

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

// out = table[src] over the rows layout (see map_rows_kernel): FLAT, or an innermost dimension that
// is a multiple of the 8-element chunk below up to 5 outer dimensions.
template <bool FLAT>
__global__ void __launch_bounds__(kTableBlock) map_table_kernel(RowsArgs<2> a, const uint16_t *table) {
    constexpr int V = 8, U = 4;
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
                u32x4 res;
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const uint32_t w = raw[u][j];
                    res[j] = static_cast<uint32_t>(lut[w & 0xFFFFu]) | (static_cast<uint32_t>(lut[w >> 16]) << 16);
                }
                *reinterpret_cast<u32x4 *>(a.ptr[0] + static_cast<int64_t>(oo[u]) * 2) = res;
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

template <class F>
void launch_table(const MapCall &c, uint16_t *table, hipStream_t stream) {
    const int variant = resolve_variant<F>(c);
    RowsArgs<2> a = rows_args<F>(c, variant);
    const int64_t tiles = (c.n + 7) / 8;
    int64_t blocks = (tiles + 4 * kTableBlock - 1) / (4 * kTableBlock);
    if (blocks > c.compute_units) blocks = c.compute_units;  // one resident workgroup per CU, each loops
    if (variant == 0) {
        hipLaunchKernelGGL((map_table_kernel<true>), dim3(static_cast<unsigned>(blocks)), dim3(kTableBlock), 0, stream, a, table);
    } else {
        hipLaunchKernelGGL((map_table_kernel<false>), dim3(static_cast<unsigned>(blocks)), dim3(kTableBlock), 0, stream, a, table);
    }
}

}  // namespace hmr
