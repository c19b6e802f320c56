// A stable least-significant-digit radix sort of 64-bit words by a field of their high halves, for the
// deterministic adds of the indexing kernels: word = (target << 32) | position, positions ascending on input, so
// sorting stably by the target's bits alone leaves every target's positions in order.
//
// A pass handles 8 bits. Workgroups take tiles of 2048 words:
//   count    the tile's digit histogram into hist[digit][tile] (digit-major, so that one exclusive scan of the whole
//            table gives, for every digit and tile, where the tile's words of that digit go);
//   scan     the table in chunks of 4096 entries, then the chunks' totals by one workgroup (sorts of up to 16 tiles
//            skip both: their scatter workgroups add up the small table themselves);
//   scatter  the tile again: every word's rank among the tile's words of its digit, in input order (waves find
//            their equal digits with ballots, the counts per round and wave are scanned in LDS), the words placed
//            in LDS in sorted order, and written out from there so that runs of a digit leave as whole lines.
// Nothing depends on the order in which workgroups or waves run: counts are sums, ranks are positions.
#pragma once

#include "ew_common.hpp"

namespace hmr {

constexpr int kSortThreads = 256;
constexpr int kSortRounds = 8;  // words per thread (4 and 16 measured slower)
constexpr int kSortTile = kSortThreads * kSortRounds;
constexpr int kSortDigits = 256;
constexpr int kSortWaves = kSortThreads / 64;
constexpr int kSortScanChunk = 4096;
constexpr int kSortScanBlock = 1024;

// The workspace of a sort of n words: [words A][words B][hist: 256 x tiles u32][totals: chunks u32].
struct SortLayout {
    int64_t n, tiles, entries, chunks;
    int64_t off_b, off_hist, off_totals, bytes;
};

inline SortLayout sort_layout(int64_t n) {
    SortLayout l{};
    l.n = n;
    l.tiles = (n + kSortTile - 1) / kSortTile;
    l.entries = l.tiles * kSortDigits;
    l.chunks = (l.entries + kSortScanChunk - 1) / kSortScanChunk;
    l.off_b = n * 8;
    l.off_hist = 2 * n * 8;
    l.off_totals = l.off_hist + l.entries * 4;
    l.bytes = (l.off_totals + l.chunks * 4 + 255) / 256 * 256;
    return l;
}

// The lanes of the wave whose digit equals this lane's, among the lanes in `valid`.
__device__ __forceinline__ uint64_t same_digit(uint32_t digit, uint64_t valid) {
    uint64_t peers = valid;
#pragma unroll
    for (int b = 0; b < 8; ++b) {
        const uint64_t set = __builtin_amdgcn_ballot_w64((digit >> b) & 1u);
        peers &= ((digit >> b) & 1u) ? set : ~set;
    }
    return peers;
}

__device__ __forceinline__ uint32_t lanes_below(uint64_t mask) {
    return __builtin_amdgcn_mbcnt_hi(static_cast<uint32_t>(mask >> 32), __builtin_amdgcn_mbcnt_lo(static_cast<uint32_t>(mask), 0u));
}

static __global__ void __launch_bounds__(kSortThreads) radix_count_kernel(const uint64_t *words, int64_t n, int shift, uint32_t *hist,
                                                                   int64_t tiles) {
    __shared__ uint32_t counts[kSortDigits];
    counts[threadIdx.x] = 0;
    __syncthreads();
    const int64_t base = static_cast<int64_t>(blockIdx.x) * kSortTile;
    uint64_t word[kSortRounds];
#pragma unroll
    for (int r = 0; r < kSortRounds; ++r) {  // every load is out before the first ballot waits for one
        const int64_t i = base + r * kSortThreads + threadIdx.x;
        word[r] = i < n ? words[i] : 0;
    }
#pragma unroll
    for (int r = 0; r < kSortRounds; ++r) {
        const int64_t i = base + r * kSortThreads + threadIdx.x;
        const bool valid = i < n;
        const uint64_t lanes = __builtin_amdgcn_ballot_w64(valid);
        if (valid) {
            const uint32_t digit = static_cast<uint32_t>(word[r] >> shift) & 0xFFu;
            const uint64_t peers = same_digit(digit, lanes);
            if (lanes_below(peers) == 0) atomicAdd(&counts[digit], static_cast<uint32_t>(__popcll(peers)));
        }
    }
    __syncthreads();
    hist[static_cast<int64_t>(threadIdx.x) * tiles + blockIdx.x] = counts[threadIdx.x];
}

// Exclusive prefix sums inside each chunk of 4096 entries; the chunk's sum goes to totals[chunk].
static __global__ void __launch_bounds__(kSortThreads) scan_chunks_kernel(uint32_t *a, int64_t len, uint32_t *totals) {
    constexpr int kPer = kSortScanChunk / kSortThreads;
    __shared__ uint32_t lds[kSortWaves];
    const int lane = threadIdx.x & 63, wave = threadIdx.x / 64;
    const int64_t first = static_cast<int64_t>(blockIdx.x) * kSortScanChunk + static_cast<int64_t>(threadIdx.x) * kPer;
    uint32_t v[kPer];
    uint32_t sum = 0;
#pragma unroll
    for (int i = 0; i < kPer; ++i) {
        v[i] = first + i < len ? a[first + i] : 0u;
        sum += v[i];
    }
    uint32_t x = sum;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
        const uint32_t y = static_cast<uint32_t>(__shfl_up(static_cast<int>(x), off, 64));
        if (lane >= off) x += y;
    }
    if (lane == 63) lds[wave] = x;
    __syncthreads();
    uint32_t before = x - sum;
    for (int w = 0; w < wave; ++w) before += lds[w];
#pragma unroll
    for (int i = 0; i < kPer; ++i) {
        if (first + i < len) a[first + i] = before;
        before += v[i];
    }
    if (threadIdx.x == kSortThreads - 1) totals[blockIdx.x] = before;
}

// One workgroup: totals become their exclusive prefix sums.
static __global__ void __launch_bounds__(kSortScanBlock) scan_totals_kernel(uint32_t *totals, int64_t chunks) {
    __shared__ uint32_t lds[kSortScanBlock / 64];
    const int lane = threadIdx.x & 63, wave = threadIdx.x / 64;
    uint32_t carry = 0;
    for (int64_t base = 0; base < chunks; base += kSortScanBlock) {
        const int64_t i = base + threadIdx.x;
        const uint32_t v = i < chunks ? totals[i] : 0u;
        uint32_t x = v;
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
            const uint32_t y = static_cast<uint32_t>(__shfl_up(static_cast<int>(x), off, 64));
            if (lane >= off) x += y;
        }
        if (lane == 63) lds[wave] = x;
        __syncthreads();
        uint32_t before = 0, total = 0;
        for (int w = 0; w < kSortScanBlock / 64; ++w) {
            before += w < wave ? lds[w] : 0u;
            total += lds[w];
        }
        if (i < chunks) totals[i] = carry + before + x - v;
        carry += total;
        __syncthreads();
    }
}

// SELF_SCAN: `hist` is the table as radix_count_kernel left it, of at most kSortSelfTiles tiles, and every workgroup
// finds its own places in it: thread d adds up digit d's counts over the tiles (the digit's words, and those of the
// tiles before this one), the digits' sums are scanned over the workgroup. Two launches fewer per pass, which for a
// sort of some ten thousand words is a third of its time.
constexpr int kSortSelfTiles = 16;
template <bool SELF_SCAN>
static __global__ void __launch_bounds__(kSortThreads) radix_scatter_kernel(const uint64_t *in, uint64_t *out, int64_t n, int shift,
                                                                     const uint32_t *hist, const uint32_t *totals, int64_t tiles) {
    __shared__ uint16_t counts[kSortRounds][kSortWaves][kSortDigits];  // words of a digit in (round, wave), then their prefix
    __shared__ uint64_t sorted[kSortTile];
    __shared__ uint32_t digit_base[kSortDigits];  // where the tile's words of a digit start in `out`, minus local_base
    __shared__ uint32_t local_base[kSortDigits];  // ... and in `sorted`
    __shared__ uint32_t wave_sums[kSortWaves];
    const int lane = threadIdx.x & 63, wave = threadIdx.x / 64;
    uint32_t *zero = reinterpret_cast<uint32_t *>(&counts[0][0][0]);
    for (int i = threadIdx.x; i < kSortRounds * kSortWaves * kSortDigits / 2; i += kSortThreads) zero[i] = 0;
    __syncthreads();
    const int64_t base = static_cast<int64_t>(blockIdx.x) * kSortTile;
    const int64_t left = n - base;
    const uint32_t in_tile = left < kSortTile ? static_cast<uint32_t>(left) : static_cast<uint32_t>(kSortTile);
    uint64_t word[kSortRounds];
    uint32_t rank[kSortRounds];  // among the wave's words of the digit in this round
#pragma unroll
    for (int r = 0; r < kSortRounds; ++r) {
        const uint32_t j = r * kSortThreads + threadIdx.x;
        const bool valid = j < in_tile;
        const uint64_t lanes = __builtin_amdgcn_ballot_w64(valid);
        word[r] = valid ? in[base + j] : 0;
        rank[r] = 0;
        if (valid) {
            const uint32_t digit = static_cast<uint32_t>(word[r] >> shift) & 0xFFu;
            const uint64_t peers = same_digit(digit, lanes);
            rank[r] = lanes_below(peers);
            if (rank[r] == 0) counts[r][wave][digit] = static_cast<uint16_t>(__popcll(peers));
        }
    }
    __syncthreads();
    // Thread d: the prefix of digit d's counts over (round, wave) in input order, and the digit's total.
    uint32_t running = 0;
#pragma unroll 4
    for (int r = 0; r < kSortRounds; ++r) {
#pragma unroll
        for (int w = 0; w < kSortWaves; ++w) {
            const uint32_t c = counts[r][w][threadIdx.x];
            counts[r][w][threadIdx.x] = static_cast<uint16_t>(running);
            running += c;
        }
    }
    // Exclusive scan of the digits' totals over the workgroup.
    uint32_t x = running;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
        const uint32_t y = static_cast<uint32_t>(__shfl_up(static_cast<int>(x), off, 64));
        if (lane >= off) x += y;
    }
    if (lane == 63) wave_sums[wave] = x;
    __syncthreads();
    uint32_t before = x - running;
    for (int w = 0; w < wave; ++w) before += wave_sums[w];
    const int64_t entry = static_cast<int64_t>(threadIdx.x) * tiles + blockIdx.x;
    local_base[threadIdx.x] = before;
    if constexpr (SELF_SCAN) {
        uint32_t all = 0, ahead = 0;  // digit threadIdx.x: its words in every tile, and in the tiles before this one
        for (int t = 0; t < static_cast<int>(tiles); ++t) {
            const uint32_t c = hist[static_cast<int64_t>(threadIdx.x) * tiles + t];
            all += c;
            ahead += t < static_cast<int>(blockIdx.x) ? c : 0u;
        }
        uint32_t y = all;
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
            const uint32_t z = static_cast<uint32_t>(__shfl_up(static_cast<int>(y), off, 64));
            if (lane >= off) y += z;
        }
        __syncthreads();  // wave_sums was read above
        if (lane == 63) wave_sums[wave] = y;
        __syncthreads();
        uint32_t smaller = y - all;  // words of smaller digits, in all tiles
        for (int w = 0; w < wave; ++w) smaller += wave_sums[w];
        digit_base[threadIdx.x] = smaller + ahead - before;
    } else {
        digit_base[threadIdx.x] = hist[entry] + totals[entry / kSortScanChunk] - before;
    }
    __syncthreads();
#pragma unroll
    for (int r = 0; r < kSortRounds; ++r) {
        const uint32_t j = r * kSortThreads + threadIdx.x;
        if (j < in_tile) {
            const uint32_t digit = static_cast<uint32_t>(word[r] >> shift) & 0xFFu;
            sorted[local_base[digit] + counts[r][wave][digit] + rank[r]] = word[r];
        }
    }
    __syncthreads();
    for (uint32_t j = threadIdx.x; j < in_tile; j += kSortThreads) {
        const uint64_t w = sorted[j];
        out[digit_base[static_cast<uint32_t>(w >> shift) & 0xFFu] + j] = w;
    }
}

// Sorts the n words at the start of `workspace` (sort_layout(n).bytes of it) by bits [32, 32 + key_bits) of
// each, stably, and returns where the sorted words are (the start of the workspace or its second buffer).
inline uint64_t *sort_words(void *workspace, int64_t n, int key_bits, hipStream_t stream) {
    const SortLayout l = sort_layout(n);
    char *p = static_cast<char *>(workspace);
    uint64_t *a = reinterpret_cast<uint64_t *>(p), *b = reinterpret_cast<uint64_t *>(p + l.off_b);
    uint32_t *hist = reinterpret_cast<uint32_t *>(p + l.off_hist), *totals = reinterpret_cast<uint32_t *>(p + l.off_totals);
    for (int done = 0; done < key_bits; done += 8) {
        const int shift = 32 + done;
        const dim3 grid(static_cast<unsigned>(l.tiles));
        hipLaunchKernelGGL(radix_count_kernel, grid, dim3(kSortThreads), 0, stream, static_cast<const uint64_t *>(a), n, shift, hist, l.tiles);
        if (l.tiles <= kSortSelfTiles) {
            hipLaunchKernelGGL(radix_scatter_kernel<true>, grid, dim3(kSortThreads), 0, stream, static_cast<const uint64_t *>(a), b, n,
                               shift, static_cast<const uint32_t *>(hist), static_cast<const uint32_t *>(totals), l.tiles);
        } else {
            hipLaunchKernelGGL(scan_chunks_kernel, dim3(static_cast<unsigned>(l.chunks)), dim3(kSortThreads), 0, stream, hist, l.entries,
                               totals);
            hipLaunchKernelGGL(scan_totals_kernel, dim3(1), dim3(kSortScanBlock), 0, stream, totals, l.chunks);
            hipLaunchKernelGGL(radix_scatter_kernel<false>, grid, dim3(kSortThreads), 0, stream, static_cast<const uint64_t *>(a), b, n,
                               shift, static_cast<const uint32_t *>(hist), static_cast<const uint32_t *>(totals), l.tiles);
        }
        uint64_t *t = a;
        a = b;
        b = t;
    }
    return a;
}

// Bits needed for values 0 .. max_value.
inline int bits_for(uint64_t max_value) {
    int bits = 0;
    while (bits < 64 && (max_value >> bits) != 0) ++bits;
    return bits;
}

}  // namespace hmr
