// hmr_index_check, hmr_index_select, hmr_gather, hmr_index_add(+workspace), hmr_scatter_add(+workspace)
// (ref: csrc/homura_rocm.h:353-404, csrc/index.hip; the semantics are src/backend/cpu/misc.rs:53-127, 213-345).
//
// Index tensors are I32 or I64. The caller checks positions first (hmr_index_check in the same
// critical section), so the other kernels take them as valid.
//   reads   index_select copies rows of 16-byte tiles when the slices are contiguous (an embedding
//           lookup: one index load and one row offset per tile, the rest is a copy) and single elements
//           otherwise; gather is one element per thread.
//   adds    every element of the output is summed in f64 (wrapping i64 for integers) in the row-major
//           order of the index positions and rounded once, as the CPU does. Addition is not
//           associative, so the order is reproduced: each contribution becomes a 64-bit word
//           (target << 32 | position), the words are sorted by target with a stable radix sort (sort.hpp;
//           positions ascend on input, so each target's stay in order), and the first word of each target
//           sums its run in order. Targets run in parallel; index_add also spreads a slice over the lanes.
#include "mail.hpp"
#include "index.hpp"
#include "sort.hpp"

namespace hmr {
namespace {

// ---- hmr_index_check ------------------------------------------------------------------------------------

// A check is ONE launch. Its workgroups meet in `CheckState` (device memory of the context): every wave that
// found a bad position lowers `first` (a minimum does not depend on the order they arrive in), every workgroup
// then counts itself in, and the one that arrives last reads the minimum, looks the value at that position up,
// publishes both - in the caller's slot and in the context's mailbox (pinned host memory, so that the caller's
// read-back is a wait for the stream and nothing else) - and leaves the state as it found it.
//
// Counting in is two levels deep: an atomic on one address costs some 16 ns however many workgroups issue it
// (2048 of them on one counter added 33 us to a check of 8.4 M positions), so a workgroup counts itself into one
// of 32 counters, each on a cache line of its own, and the last one of each counter counts into the top one.
constexpr int kCheckGroups = 32;
constexpr unsigned kCheckGrid = 1024;  // workgroups of a check at most (its kernels stride over the rest)
struct CheckState {
    unsigned long long first;  // all ones: none
    char pad0[120];
    unsigned int top;
    char pad1[124];
    struct {
        unsigned int arrived;
        char pad[124];
    } group[kCheckGroups];
};
static_assert(sizeof(CheckState) <= kCheckStateBytes, "the context keeps kCheckStateBytes for it");

__device__ __forceinline__ int64_t value_at(const void *index, int is64, const Dims &d, unsigned long long p) {
    int64_t rest = static_cast<int64_t>(p), off = 0;
    for (int k = 0; k < d.ndim; ++k) {
        const int64_t q = rest / d.size[k];
        off += (rest - q * d.size[k]) * d.stride[0][k];
        rest = q;
    }
    return read_index(index, is64, off);
}

// The verdict goes to the caller's slot and to the mailbox (mail.hpp).
__device__ __forceinline__ void publish(uint64_t *slot, uint64_t *mailbox, unsigned long long first, int64_t value, uint64_t ticket) {
    const uint64_t word = first == ~0ull ? 0 : static_cast<uint64_t>(value);
    slot[0] = first;
    slot[1] = word;
    post(mailbox, ticket, static_cast<uint64_t>(first), word);
}

// `first`: the smallest bad position this lane saw. Every lane of the workgroup calls this, once.
__device__ __forceinline__ void meet(unsigned long long first, CheckState *state, uint64_t *slot, uint64_t *mailbox,
                                     uint64_t ticket, const void *index, int is64, const Dims &d) {
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) {
        const unsigned long long other = (static_cast<unsigned long long>(static_cast<uint32_t>(__shfl_xor(static_cast<int>(first >> 32), m, 64))) << 32) |
                                         static_cast<uint32_t>(__shfl_xor(static_cast<int>(first), m, 64));
        first = other < first ? other : first;
    }
    if ((threadIdx.x & 63) == 0 && first != ~0ull) atomicMin(&state->first, first);
    __syncthreads();  // every wave's minimum is out
    if (threadIdx.x != 0) return;
    const unsigned mine = blockIdx.x % kCheckGroups;
    const unsigned members = (gridDim.x - mine + kCheckGroups - 1) / kCheckGroups;
    const unsigned groups = gridDim.x < kCheckGroups ? gridDim.x : kCheckGroups;
    // No fences between these: every one of them is an atomic of device scope, carried out where all compute dies
    // see it; a wave's atomicMin has been acknowledged before the barrier above lets this lane go on, and each
    // step below is issued only after the one before it has returned its value. (A device-scope fence would write
    // back and invalidate the die's L2 once per workgroup: a check of 8.4 M positions took 25 us with them, 7 without.)
    if (atomicAdd(&state->group[mine].arrived, 1u) != members - 1) return;
    atomicExch(&state->group[mine].arrived, 0u);
    if (atomicAdd(&state->top, 1u) != groups - 1) return;
    atomicExch(&state->top, 0u);
    const unsigned long long found = atomicExch(&state->first, ~0ull);
    publish(slot, mailbox, found, found == ~0ull ? 0 : value_at(index, is64, d, found), ticket);
}

__global__ void __launch_bounds__(kBlock) check_kernel(const void *index, int is64, Dims d, int64_t n, int64_t low, int64_t high,
                                                       int has_exempt, int64_t exempt, uint64_t *slot, CheckState *state, uint64_t *mailbox, uint64_t ticket) {
    unsigned long long first = ~0ull;
    for (int64_t p = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x; p < n; p += static_cast<int64_t>(gridDim.x) * kBlock) {
        int64_t rest = p, off = p * d.stride[0][0];
        if (d.ndim > 1) {
            off = 0;
            for (int k = 0; k < d.ndim; ++k) {
                const int64_t q = rest / d.size[k];
                off += (rest - q * d.size[k]) * d.stride[0][k];
                rest = q;
            }
        }
        const int64_t v = read_index(index, is64, off);
        const bool bad = !(v >= low && v < high) && !(has_exempt && v == exempt);
        if (bad && static_cast<unsigned long long>(p) < first) first = static_cast<unsigned long long>(p);
    }
    meet(first, state, slot, mailbox, ticket, index, is64, d);
}

// The same for an index that is one contiguous run: 16 bytes per lane and load, four loads in flight (an
// element per lane reads 33 MB of positions in 22 us; this form in a third of that). `head` elements (fewer
// than a tile) come before the first 16-byte boundary; they and the ragged end go to the first workgroup's lanes.
template <class I>
__global__ void __launch_bounds__(kBlock) check_flat_kernel(const I *start, int head, int64_t total, int64_t low, int64_t high,
                                                            int has_exempt, int64_t exempt, uint64_t *slot, CheckState *state, uint64_t *mailbox, uint64_t ticket,
                                                            Dims d) {
    constexpr int V = 16 / static_cast<int>(sizeof(I)), U = 4;
    unsigned long long first = ~0ull;
    const I *index = start + head;  // aligned; position p of the run is index[p - head]
    const int64_t n = total - head;
    const int64_t tiles = n / V;
    for (int64_t t0 = static_cast<int64_t>(blockIdx.x) * (U * kBlock) + threadIdx.x; t0 < tiles;
         t0 += static_cast<int64_t>(gridDim.x) * (U * kBlock)) {
        I v[U][V];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int64_t t = t0 + static_cast<int64_t>(u) * kBlock;
            load_tile<I, V, true>(reinterpret_cast<const char *>(index + (t < tiles ? t : tiles - 1) * V), v[u]);
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int64_t t = t0 + static_cast<int64_t>(u) * kBlock;
#pragma unroll
            for (int i = V - 1; i >= 0; --i) {  // backwards: the smallest position of the tile ends up in `first`
                const int64_t x = static_cast<int64_t>(v[u][i]);
                const bool bad = t < tiles && !(x >= low && x < high) && !(has_exempt && x == exempt);
                const unsigned long long p = static_cast<unsigned long long>(t * V + i + head);
                if (bad && p < first) first = p;
            }
        }
    }
    // The head and the ragged end (fewer than V elements each), by the first lanes of the first workgroup.
    if (blockIdx.x == 0) {
        const int64_t tail = n - tiles * V;
        int64_t p = -1;
        if (threadIdx.x < static_cast<unsigned>(head)) p = threadIdx.x;
        else if (threadIdx.x - head < tail) p = head + tiles * V + (threadIdx.x - head);
        if (p >= 0) {
            const int64_t x = static_cast<int64_t>(start[p]);
            if (!(x >= low && x < high) && !(has_exempt && x == exempt) && static_cast<unsigned long long>(p) < first) first = p;
        }
    }
    meet(first, state, slot, mailbox, ticket, start, sizeof(I) == 8, d);
}

// The whole check in one workgroup, for indices of a few thousand elements: no meeting, no atomics.
constexpr int kCheckBlock = 1024;
constexpr int64_t kCheckSmall = 16 * kCheckBlock;
__global__ void __launch_bounds__(kCheckBlock) check_small_kernel(const void *index, int is64, Dims d, int64_t n, int64_t low, int64_t high,
                                                                  int has_exempt, int64_t exempt, uint64_t *slot, uint64_t *mailbox, uint64_t ticket) {
    __shared__ unsigned long long firsts[kCheckBlock / 64];
    __shared__ long long values[kCheckBlock / 64];
    unsigned long long first = ~0ull;
    long long value = 0;
    constexpr int kAhead = 8;  // loads in flight per lane
    for (int64_t p0 = threadIdx.x; p0 < n; p0 += static_cast<int64_t>(kAhead) * kCheckBlock) {
        int64_t v[kAhead];
#pragma unroll
        for (int u = 0; u < kAhead; ++u) {
            const int64_t p = p0 + static_cast<int64_t>(u) * kCheckBlock;
            const int64_t q = p < n ? p : n - 1;  // past the end: the last element again, left out below
            int64_t rest = q, off = q * d.stride[0][0];
            if (d.ndim > 1) {
                off = 0;
                for (int k = 0; k < d.ndim; ++k) {
                    const int64_t w = rest / d.size[k];
                    off += (rest - w * d.size[k]) * d.stride[0][k];
                    rest = w;
                }
            }
            v[u] = read_index(index, is64, off);
        }
#pragma unroll
        for (int u = 0; u < kAhead; ++u) {
            const int64_t p = p0 + static_cast<int64_t>(u) * kCheckBlock;
            const bool bad = p < n && !(v[u] >= low && v[u] < high) && !(has_exempt && v[u] == exempt);
            if (bad && static_cast<unsigned long long>(p) < first) {
                first = static_cast<unsigned long long>(p);
                value = v[u];
            }
        }
    }
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) {
        const unsigned long long other = (static_cast<unsigned long long>(static_cast<uint32_t>(__shfl_xor(static_cast<int>(first >> 32), m, 64))) << 32) |
                                         static_cast<uint32_t>(__shfl_xor(static_cast<int>(first), m, 64));
        const long long theirs = static_cast<long long>((static_cast<unsigned long long>(static_cast<uint32_t>(__shfl_xor(static_cast<int>(value >> 32), m, 64))) << 32) |
                                                        static_cast<uint32_t>(__shfl_xor(static_cast<int>(value), m, 64)));
        if (other < first) {
            first = other;
            value = theirs;
        }
    }
    if ((threadIdx.x & 63) == 0) {
        firsts[threadIdx.x / 64] = first;
        values[threadIdx.x / 64] = value;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < kCheckBlock / 64; ++w) {
            if (firsts[w] < first) {
                first = firsts[w];
                value = values[w];
            }
        }
        publish(slot, mailbox, first, value, ticket);
    }
}

__global__ void check_value_kernel(const void *index, int is64, Dims d, uint64_t *slot) {
    const uint64_t p = slot[0];
    if (p == ~uint64_t{0}) return;
    slot[1] = static_cast<uint64_t>(value_at(index, is64, d, p));
}

// ---- hmr_index_select / hmr_gather ---------------------------------------------------------------------

// One element per thread. stride[0] out, [1] src, [2] the index (gather: walked like out; index_select:
// only along `at`). `wrap` adds the source's size along `at` to a negative position.
template <class W>
__global__ void __launch_bounds__(kBlock) pick_kernel(W *out, const W *src, const void *index, int is64, Dims d, int64_t n,
                                                      int64_t wrap) {
    // Four picks per lane, a workgroup apart: their positions are read first, then their elements, then they are
    // stored (one pick per lane leaves a wave with one dependent pair of loads in flight; eight were no faster).
    // The outermost dimension needs no division.
    constexpr int U = 4;
    for (int64_t base = static_cast<int64_t>(blockIdx.x) * (U * kBlock); base < n; base += static_cast<int64_t>(gridDim.x) * (U * kBlock)) {
        int64_t oo[U], so[U], j[U];
        bool valid[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int64_t wanted = base + static_cast<int64_t>(u) * kBlock + threadIdx.x;
            valid[u] = wanted < n;
            int64_t rest = valid[u] ? wanted : n - 1, io = 0;
            oo[u] = so[u] = 0;
            for (int k = 0; k < d.ndim; ++k) {
                int64_t c = rest;
                if (k + 1 < d.ndim) {
                    // n is below 2^32 for all but the largest tensors: a 32-bit division is a third of a 64-bit one.
                    const int64_t q = n <= int64_t{0xFFFFFFFF} ? static_cast<int64_t>(static_cast<uint32_t>(rest) / static_cast<uint32_t>(d.size[k]))
                                                               : rest / d.size[k];
                    c = rest - q * d.size[k];
                    rest = q;
                }
                oo[u] += c * d.stride[0][k];
                io += c * d.stride[2][k];
                if (k != d.at) so[u] += c * d.stride[1][k];
            }
            j[u] = read_index(index, is64, io);
        }
        W v[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            if (j[u] < 0) j[u] += wrap;
            v[u] = src[so[u] + j[u] * d.stride[1][d.at]];
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            if (!valid[u]) continue;
            // Results too large for the caches to keep for a reader go past them, as everywhere in the library.
            if (n * static_cast<int64_t>(sizeof(W)) >= kStreamStoreBytes) __builtin_nontemporal_store(v[u], out + oo[u]);
            else out[oo[u]] = v[u];
        }
    }
}

// index_select of contiguous slices: the innermost dimension is a run of whole 16-byte tiles in both
// operands; the dimensions outside it (the indexed one among them) are decomposed once per tile.
struct RowsOfTiles {
    char *out;
    const char *src;
    const void *index;
    int32_t is64, nouter, at;  // `at` counts outer dimensions from the innermost outer one
    int32_t out32;             // nonzero: every byte offset into the output fits 32 bits
    int64_t n_tiles, wrap, index_stride;
    uint32_t tiles_per_row;
    FastDiv tiles_div;
    FastDiv div[kMaxIndexDims];
    int64_t stride[2][kMaxIndexDims];  // of the outer dimensions, in elements
};

template <class W>
__global__ void __launch_bounds__(kBlock) select_rows_kernel(RowsOfTiles a) {
    constexpr int V = 16 / static_cast<int>(sizeof(W));
    constexpr int U = 4;
    const OutStores stores(a.out, a.out32 != 0);
    const int64_t first = static_cast<int64_t>(blockIdx.x) * (U * kBlock) + threadIdx.x;
    W r[U][V];
    int64_t oo[U];
    bool valid[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
        const int64_t t = first + static_cast<int64_t>(u) * kBlock;
        valid[u] = t < a.n_tiles;
        const uint32_t tt = static_cast<uint32_t>(valid[u] ? t : a.n_tiles - 1);
        uint32_t row = divide(tt, a.tiles_div);
        const int64_t col = static_cast<int64_t>(tt - row * a.tiles_per_row) * V;
        int64_t o = col, s = col;
        for (int k = 0; k < a.nouter; ++k) {
            const uint32_t q = divide(row, a.div[k]);
            const int64_t c = row - q * a.div[k].div;
            row = q;
            o += c * a.stride[0][k];
            if (k == a.at) {
                int64_t j = read_index(a.index, a.is64, c * a.index_stride);
                if (j < 0) j += a.wrap;
                s += j * a.stride[1][k];
            } else {
                s += c * a.stride[1][k];
            }
        }
        oo[u] = o;
        load_tile<W, V, kStreamLoads>(a.src + s * static_cast<int64_t>(sizeof(W)), r[u]);
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int u = 0; u < U; ++u) {
        if (valid[u]) {
            u32x4 w;
            __builtin_memcpy(&w, r[u], 16);
            stores.put16(oo[u] * static_cast<int64_t>(sizeof(W)), w);
        }
    }
}

// ---- adds ---------------------------------------------------------------------------------------------------

template <class T>
struct Sum {
    static constexpr bool kFloat = Conv<T>::kind == Kind::Float;
    using A = std::conditional_t<kFloat, double, int64_t>;
    static __device__ __forceinline__ A widen(T x) {
        if constexpr (kFloat) return Conv<T>::to_f64(x);
        else return Conv<T>::to_i64(x);
    }
    static __device__ __forceinline__ A add(A acc, T x) {
        if constexpr (kFloat) return acc + Conv<T>::to_f64(x);
        else return static_cast<int64_t>(static_cast<uint64_t>(acc) + static_cast<uint64_t>(Conv<T>::to_i64(x)));
    }
    static __device__ __forceinline__ T narrow(A acc) {
        if constexpr (kFloat) return Conv<T>::from_f64(acc);
        else return Conv<T>::from_i64(acc);
    }
};

// scatter_add: word p = (offset of the target in out << 32) | p, for the index's positions p in row-major
// order; stride[0] the index, [1] out (its stride along `at` multiplies the index value), [2] src.
__global__ void __launch_bounds__(kBlock) scatter_words_kernel(uint64_t *words, const void *index, int is64, Dims d, int64_t n) {
    for (int64_t p = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x; p < n; p += static_cast<int64_t>(gridDim.x) * kBlock) {
        int64_t rest = p, io = 0, oo = 0;
        for (int k = 0; k < d.ndim; ++k) {
            const int64_t q = rest / d.size[k];
            const int64_t c = rest - q * d.size[k];
            rest = q;
            io += c * d.stride[0][k];
            if (k != d.at) oo += c * d.stride[1][k];
        }
        oo += read_index(index, is64, io) * d.stride[1][d.at];
        words[p] = (static_cast<uint64_t>(oo) << 32) | static_cast<uint64_t>(p);
    }
}

template <class T>
__global__ void __launch_bounds__(kBlock) scatter_runs_kernel(T *out, const T *src, const uint64_t *words, Dims d, int64_t n) {
    using S = Sum<T>;
    for (int64_t r = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x; r < n; r += static_cast<int64_t>(gridDim.x) * kBlock) {
        const uint64_t target = words[r] >> 32;
        if (r > 0 && (words[r - 1] >> 32) == target) continue;  // not the first of its run
        typename S::A acc = S::widen(out[target]);
        for (int64_t e = r; e < n; ++e) {
            const uint64_t w = words[e];
            if ((w >> 32) != target) break;
            int64_t rest = static_cast<int64_t>(w & 0xFFFFFFFFu), so = 0;
            for (int k = 0; k < d.ndim; ++k) {
                const int64_t q = rest / d.size[k];
                so += (rest - q * d.size[k]) * d.stride[2][k];
                rest = q;
            }
            acc = S::add(acc, src[so]);
        }
        out[target] = S::narrow(acc);
    }
}

// index_add: word i = (index[i] << 32) | i.
__global__ void __launch_bounds__(kBlock) index_words_kernel(uint64_t *words, const void *index, int is64, int64_t index_stride,
                                                             int64_t m) {
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x; i < m; i += static_cast<int64_t>(gridDim.x) * kBlock) {
        words[i] = (static_cast<uint64_t>(read_index(index, is64, i * index_stride)) << 32) | static_cast<uint64_t>(i);
    }
}

// A group of `lanes` threads (a power of two up to the workgroup) takes one sorted word; the group of a
// run's first word sums the run for the elements of the slice, which its lanes share out. `d` holds
// the slice's dimensions (every dimension but the indexed one): stride[0] out, [1] src.
template <class T>
__global__ void __launch_bounds__(kBlock) index_runs_kernel(T *out, const T *src, const uint64_t *words, Dims d, int64_t m,
                                                            int64_t slice, int64_t out_step, int64_t src_step, int lanes) {
    using S = Sum<T>;
    const int per_block = kBlock / lanes;
    const int lane = threadIdx.x % lanes;
    for (int64_t r = static_cast<int64_t>(blockIdx.x) * per_block + threadIdx.x / lanes; r < m;
         r += static_cast<int64_t>(gridDim.x) * per_block) {
        const uint64_t target = words[r] >> 32;
        if (r > 0 && (words[r - 1] >> 32) == target) continue;
        for (int64_t e = lane; e < slice; e += lanes) {
            int64_t rest = e, oo = 0, so = 0;
            for (int k = 0; k < d.ndim; ++k) {
                const int64_t q = rest / d.size[k];
                const int64_t c = rest - q * d.size[k];
                rest = q;
                oo += c * d.stride[0][k];
                so += c * d.stride[1][k];
            }
            T *po = out + oo + static_cast<int64_t>(target) * out_step;
            typename S::A acc = S::widen(*po);
            for (int64_t x = r; x < m; ++x) {
                const uint64_t w = words[x];
                if ((w >> 32) != target) break;
                acc = S::add(acc, src[so + static_cast<int64_t>(w & 0xFFFFFFFFu) * src_step]);
            }
            *po = S::narrow(acc);
        }
    }
}

// The same when a slice is one contiguous run of whole aligned 16-byte tiles in both operands (the rows of
// an embedding table): a lane owns a tile and keeps its V sums in registers.
template <class T>
__global__ void __launch_bounds__(kBlock) index_runs_tiles_kernel(T *out, const T *src, const uint64_t *words, int64_t m,
                                                                  int64_t tiles, int64_t out_step, int64_t src_step, int lanes) {
    using S = Sum<T>;
    constexpr int V = 16 / static_cast<int>(sizeof(T));
    const int per_block = kBlock / lanes;
    const int lane = threadIdx.x % lanes;
    for (int64_t r = static_cast<int64_t>(blockIdx.x) * per_block + threadIdx.x / lanes; r < m;
         r += static_cast<int64_t>(gridDim.x) * per_block) {
        const uint64_t first = words[r];
        const uint64_t target = first >> 32;
        if (r > 0 && (words[r - 1] >> 32) == target) continue;
        // Two tiles of the row per step, and for each the target's tile and the run's first source tile requested
        // together: most runs are one row long, and a lane's chain is then the sorted word, these loads, the store
        // (one tile at a time with the source behind the target it was three round trips per tile).
        constexpr int U = 2;
        const int64_t from = static_cast<int64_t>(first & 0xFFFFFFFFu) * src_step;
        for (int64_t t0 = lane; t0 < tiles; t0 += static_cast<int64_t>(U) * lanes) {
            T v[U][V], s0[U][V];
            typename S::A acc[U][V];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int64_t t = t0 + static_cast<int64_t>(u) * lanes < tiles ? t0 + static_cast<int64_t>(u) * lanes : t0;
                load_tile<T, V, false>(reinterpret_cast<const char *>(out + static_cast<int64_t>(target) * out_step + t * V), v[u]);
                load_tile<T, V, false>(reinterpret_cast<const char *>(src + from + t * V), s0[u]);
            }
#pragma unroll
            for (int u = 0; u < U; ++u) {
#pragma unroll
                for (int i = 0; i < V; ++i) acc[u][i] = S::add(S::widen(v[u][i]), s0[u][i]);
            }
            for (int64_t x = r + 1; x < m; ++x) {
                const uint64_t w = words[x];
                if ((w >> 32) != target) break;
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    const int64_t t = t0 + static_cast<int64_t>(u) * lanes < tiles ? t0 + static_cast<int64_t>(u) * lanes : t0;
                    load_tile<T, V, false>(reinterpret_cast<const char *>(src + static_cast<int64_t>(w & 0xFFFFFFFFu) * src_step + t * V), s0[u]);
                }
#pragma unroll
                for (int u = 0; u < U; ++u) {
#pragma unroll
                    for (int i = 0; i < V; ++i) acc[u][i] = S::add(acc[u][i], s0[u][i]);
                }
            }
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int64_t t = t0 + static_cast<int64_t>(u) * lanes;
                if (t >= tiles) continue;
#pragma unroll
                for (int i = 0; i < V; ++i) v[u][i] = S::narrow(acc[u][i]);
                store_tile<T, V, false>(reinterpret_cast<char *>(out + static_cast<int64_t>(target) * out_step + t * V), v[u]);
            }
        }
    }
}

// ---- lines: gather and scatter_add along a dimension never leave their line -------------------------------------
//
// A line is the indexed dimension under one choice of all other coordinates. gather reads a line of the source
// at the index's positions; scatter_add adds a line of contributions into a line of the output. Lines do not
// interact, so a workgroup takes a line at a time and keeps what is accessed at random in LDS.

// Lines worth a workgroup each: enough of them to cover the GPU; scatter_add takes lines of 64 to 2048 positions
// (a word holds a position in 11 bits) into contiguous output lines of up to 64 KB, with the index and the source
// running along the line with stride 1 (their loads are coalesced then).
constexpr int64_t kMinLines = 128;
constexpr int kMaxLinePositions = 2048;
constexpr int64_t kMaxLineBytes = 65536;

// The offsets of line `line` (row-major over every dimension but `at`) in the three operands.
__device__ __forceinline__ void line_bases(const Dims &d, int64_t line, int64_t (&base)[3]) {
    base[0] = base[1] = base[2] = 0;
    for (int k = 0; k < d.ndim; ++k) {
        if (k == d.at) continue;
        const int64_t q = line / d.size[k];
        const int64_t c = line - q * d.size[k];
        line = q;
        base[0] += c * d.stride[0][k];
        base[1] += c * d.stride[1][k];
        base[2] += c * d.stride[2][k];
    }
}

// gather: the source's line (contiguous, `length` elements) is staged in LDS with coalesced loads, the picks hit
// LDS and leave as coalesced stores. stride[0] out, [1] src, [2] index; `count` positions per line; `length` is the
// source's size along the line as its description gives it.
// Every 4-byte pick straight from memory costs a 64-byte sector and one address per lane in the texture path;
// 512 picks from a 16 KB line touch nearly all of its sectors anyway.
// BYTES is the LDS a workgroup reserves (the line fits it): the smaller, the more workgroups a compute unit holds
// and the better one's load of a line hides behind another's picks.
template <class W, int BYTES>
__global__ void __launch_bounds__(kBlock) gather_lines_kernel(W *out, const W *src, const void *index, int is64, Dims d,
                                                              int64_t lines, int64_t count, int64_t length) {
    __shared__ u32x4 staged_raw[BYTES / 16];
    W *staged = reinterpret_cast<W *>(staged_raw);
    constexpr int V = 16 / static_cast<int>(sizeof(W));
    const int64_t out_step = d.stride[0][d.at], index_step = d.stride[2][d.at];
    for (int64_t line = blockIdx.x; line < lines; line += gridDim.x) {
        int64_t base[3];
        line_bases(d, line, base);
        const W *from = src + base[1];
        __syncthreads();  // the previous line's picks have read LDS
        if (reinterpret_cast<uintptr_t>(from) % 16 == 0 && length % V == 0) {
            const u32x4 *q = reinterpret_cast<const u32x4 *>(from);
            u32x4 *to = reinterpret_cast<u32x4 *>(staged);
            for (int64_t t = threadIdx.x; t < length / V; t += kBlock) to[t] = __builtin_nontemporal_load(q + t);
        } else {
            for (int64_t e = threadIdx.x; e < length; e += kBlock) staged[e] = from[e];
        }
        __syncthreads();
        W *to = out + base[0];
        for (int64_t j = threadIdx.x; j < count; j += kBlock) {
            // A caller may describe the source with the output's size along the line (only the strides matter to
            // the picks themselves): a position beyond what was staged is then read from memory.
            const int64_t at = read_index(index, is64, base[2] + j * index_step);
            to[j * out_step] = at < length ? staged[at] : from[at];
        }
    }
}

// Sorts keys[0, n) ascending in LDS, n a power of two (every thread of the workgroup calls this with the same n).
__device__ __forceinline__ void sort_in_lds(uint32_t *keys, int n) {
    for (int k = 2; k <= n; k <<= 1) {
        for (int j = k >> 1; j > 0; j >>= 1) {
            for (int i = threadIdx.x; i < n; i += kBlock) {
                const int partner = i ^ j;
                if (partner > i) {
                    const uint32_t a = keys[i], b = keys[partner];
                    const bool ascending = (i & k) == 0;
                    if ((a > b) == ascending) {
                        keys[i] = b;
                        keys[partner] = a;
                    }
                }
            }
            __syncthreads();
        }
    }
}

// scatter_add of lines of at most N positions into contiguous output lines of at most LINE_BYTES, a workgroup per
// line. The output line is staged in LDS (coalesced 16-byte loads), updated there and written back (coalesced
// stores), so memory only sees streams. Addition into an output element has to follow the order of the positions
// (the CPU's), but only where positions share a target:
//   1. two bitmaps over the output line: `seen` (some position has this target) and `multi` (a second one came:
//      atomicOr returns whether the bit was set);
//   2. a position whose target it alone holds adds its value straight into the staged element;
//   3. the others - few, unless the index repeats itself a lot - are collected as words (target << 11 | position),
//      sorted (positions are distinct, so equal targets end up in position order) and the first word of each
//      target sums its run in that order.
// f64 or wrapping i64 accumulation and one rounding per output element, as everywhere. stride[0] index, [1] out,
// [2] src. Measured on 16384 lines of 512 positions into 4096 f32 elements: every line's words (512 of 8 bytes)
// sorted whole 211 us (LDS traffic); a sort of the repeats only, with the adds going to memory element by element,
// 151 us, of which the scattered 4-byte loads and stores are 117; a wave per line no better.
template <class T, int LINE_BYTES, int N>
__global__ void __launch_bounds__(kBlock) scatter_lines_kernel(T *out, const T *src, const void *index, int is64, Dims d,
                                                               int64_t lines, int count, int length) {
    using S = Sum<T>;
    constexpr int kPositionBits = 11;
    constexpr int kMine = N / kBlock;
    constexpr int kCapacity = LINE_BYTES / static_cast<int>(sizeof(T));  // elements of a line
    constexpr int V = 16 / static_cast<int>(sizeof(T));
    __shared__ u32x4 staged_raw[LINE_BYTES / 16];
    __shared__ T values[N];  // the line's contributions, by position
    __shared__ uint32_t seen[kCapacity / 32], multi[kCapacity / 32], words[N];
    __shared__ int shared_total;
    T *staged = reinterpret_cast<T *>(staged_raw);
    const int64_t index_step = d.stride[0][d.at], src_step = d.stride[2][d.at];
    const int bitmap_words = (length + 31) / 32;
    for (int64_t line = blockIdx.x; line < lines; line += gridDim.x) {
        int64_t base[3];
        line_bases(d, line, base);
        T *to = out + base[1];
        const bool whole_tiles = reinterpret_cast<uintptr_t>(to) % 16 == 0 && length % V == 0;
        __syncthreads();  // the previous line is done with LDS
        if (whole_tiles) {
            const u32x4 *q = reinterpret_cast<const u32x4 *>(to);
            for (int t = threadIdx.x; t < length / V; t += kBlock) staged_raw[t] = q[t];
        } else {
            for (int e = threadIdx.x; e < length; e += kBlock) staged[e] = to[e];
        }
        for (int w = threadIdx.x; w < bitmap_words; w += kBlock) {
            seen[w] = 0;
            multi[w] = 0;
        }
        if (threadIdx.x == 0) shared_total = 0;
        uint32_t target[kMine];
#pragma unroll
        for (int u = 0; u < kMine; ++u) {
            const int j = threadIdx.x + u * kBlock;
            target[u] = j < count ? static_cast<uint32_t>(read_index(index, is64, base[0] + j * index_step)) : 0u;
            if (j < count) values[j] = src[base[2] + static_cast<int64_t>(j) * src_step];
        }
        __syncthreads();
#pragma unroll
        for (int u = 0; u < kMine; ++u) {
            const int j = threadIdx.x + u * kBlock;
            if (j >= count) continue;
            const uint32_t bit = 1u << (target[u] & 31u);
            if (atomicOr(&seen[target[u] >> 5], bit) & bit) atomicOr(&multi[target[u] >> 5], bit);
        }
        __syncthreads();
#pragma unroll
        for (int u = 0; u < kMine; ++u) {
            const int j = threadIdx.x + u * kBlock;
            if (j >= count) continue;
            if ((multi[target[u] >> 5] >> (target[u] & 31u)) & 1u) {
                words[atomicAdd(&shared_total, 1)] = (target[u] << kPositionBits) | static_cast<uint32_t>(j);
            } else {
                staged[target[u]] = S::narrow(S::add(S::widen(staged[target[u]]), values[j]));
            }
        }
        __syncthreads();
        const int total = shared_total;
        if (total > 0) {
            int padded = 2;
            while (padded < total) padded <<= 1;
            for (int i = total + threadIdx.x; i < padded; i += kBlock) words[i] = ~0u;
            __syncthreads();
            sort_in_lds(words, padded);
            for (int p = threadIdx.x; p < total; p += kBlock) {
                const uint32_t t = words[p] >> kPositionBits;
                if (p > 0 && (words[p - 1] >> kPositionBits) == t) continue;  // not the first of its run
                typename S::A acc = S::widen(staged[t]);
                for (int e = p; e < total; ++e) {
                    const uint32_t w = words[e];
                    if ((w >> kPositionBits) != t) break;
                    acc = S::add(acc, values[w & ((1u << kPositionBits) - 1)]);
                }
                staged[t] = S::narrow(acc);
            }
            __syncthreads();
        }
        if (whole_tiles) {
            u32x4 *q = reinterpret_cast<u32x4 *>(to);
            for (int t = threadIdx.x; t < length / V; t += kBlock) q[t] = staged_raw[t];
        } else {
            for (int e = threadIdx.x; e < length; e += kBlock) to[e] = staged[e];
        }
    }
}

}  // namespace
}  // namespace hmr

using hmr::fail;
using hmr::fenced;

extern "C" {

hmr_status hmr_index_check(hmr_context_t ctx, const hmr_tensor_desc *index, int64_t low, int64_t high, int32_t has_exempt,
                           int64_t exempt, uint64_t *slot) {
    return fenced([&] {
        int64_t n = 0;
        if (hmr_status s = hmr::check_desc(*index, n)) return s;
        if (!hmr::is_index_dtype(index->dtype)) return fail(HMR_INVALID, "index_check: unsupported dtype");
        if (slot == nullptr) return fail(HMR_INVALID, "index_check: no status slot");
        const hmr_tensor_desc *const ops[3] = {index, nullptr, nullptr};
        const hmr::Dims d = hmr::dims_of(*index, ops, -1);
        const void *base = hmr::first_of(*index);
        const int is64 = index->dtype == HMR_I64;
        if (ctx == nullptr) return fail(HMR_INVALID, "index_check: null context");
        hmr::CheckState *state = static_cast<hmr::CheckState *>(ctx->check_state);
        uint64_t *mailbox = static_cast<uint64_t *>(ctx->mailbox);
        const uint64_t ticket = ++ctx->mail_ticket;
        const hmr_status queued = hmr::queue_on(ctx, "index_check", [&](hipStream_t stream) {
            if (n <= hmr::kCheckSmall) {
                hipLaunchKernelGGL(hmr::check_small_kernel, dim3(1), dim3(hmr::kCheckBlock), 0, stream, base, is64, d, n, low, high,
                                   has_exempt, exempt, slot, mailbox, ticket);
                return true;
            }
            // One contiguous run (after merging: a size-1 dimension's stride does not count)? Its elements
            // before the first 16-byte boundary are the head.
            const int elem = is64 ? 8 : 4;
            const int64_t to_boundary = static_cast<int64_t>((16 - reinterpret_cast<uintptr_t>(base) % 16) % 16) / elem;
            const int head = static_cast<int>(to_boundary < n ? to_boundary : n);
            bool flat = reinterpret_cast<uintptr_t>(base) % elem == 0;
            int64_t run = 1;
            for (int k = index->ndim - 1; flat && k >= 0; --k) {
                flat = index->sizes[k] == 1 || index->strides[k] == run;
                run *= index->sizes[k];
            }
            if (flat) {
                const int64_t per_block = int64_t{4} * hmr::kBlock * (is64 ? 2 : 4);
                unsigned grid = hmr::grid_of((n + per_block - 1) / per_block * hmr::kBlock);
                grid = grid < hmr::kCheckGrid ? grid : hmr::kCheckGrid;
                if (is64) {
                    hipLaunchKernelGGL((hmr::check_flat_kernel<int64_t>), dim3(grid), dim3(hmr::kBlock), 0, stream,
                                       static_cast<const int64_t *>(base), head, n, low, high, has_exempt, exempt, slot, state, mailbox, ticket, d);
                } else {
                    hipLaunchKernelGGL((hmr::check_flat_kernel<int32_t>), dim3(grid), dim3(hmr::kBlock), 0, stream,
                                       static_cast<const int32_t *>(base), head, n, low, high, has_exempt, exempt, slot, state, mailbox, ticket, d);
                }
            } else {
                const unsigned all = hmr::grid_of(n);
                hipLaunchKernelGGL(hmr::check_kernel, dim3(all < hmr::kCheckGrid ? all : hmr::kCheckGrid), dim3(hmr::kBlock), 0, stream, base,
                                   is64, d, n, low, high, has_exempt, exempt, slot, state, mailbox, ticket);
            }
            return true;
        });
        // The verdict is in the mailbox as well once the kernel has run: a read-back of the slot takes it from there.
        if (queued == HMR_OK) ctx->mail_src = slot;
        return queued;
    });
}

// The second step of hmr_index_check alone (ref: csrc/homura_rocm.h:631-657, csrc/index.hip:465-479): the caller
// sets slot[0] to a logical position of `index`; unless that is UINT64_MAX the value there goes to slot[1].
// Positions reach 2^63 - 1 in views with zero strides, whose element count no longer fits 64 bits, so the
// description is checked dimension by dimension and no product is formed.
hmr_status hmr_test_index_value(hmr_context_t ctx, const hmr_tensor_desc *index, uint64_t *slot) {
    return fenced([&] {
        if (index == nullptr || slot == nullptr) return fail(HMR_INVALID, "index value: null argument");
        if (index->dtype < HMR_BOOL || index->dtype > HMR_F64) return fail(HMR_INVALID, "invalid dtype " + std::to_string(index->dtype));
        if (index->ndim < 0 || index->ndim > HMR_MAX_DIMS) {
            return fail(HMR_INVALID, "invalid number of dimensions " + std::to_string(index->ndim));
        }
        for (int k = 0; k < index->ndim; ++k) {
            if (index->sizes[k] < 0) return fail(HMR_INVALID, "negative size");
            if (index->strides[k] < 0) return fail(HMR_INVALID, "negative stride");
            if (index->sizes[k] == 0) return fail(HMR_INVALID, "index value: the index is empty");
        }
        if (!hmr::is_index_dtype(index->dtype)) return fail(HMR_INVALID, "index tensors must be I32 or I64");
        const hmr_tensor_desc *const ops[3] = {index, nullptr, nullptr};
        const hmr::Dims d = hmr::dims_of(*index, ops, -1);
        const void *base = hmr::first_of(*index);
        const int is64 = index->dtype == HMR_I64;
        return hmr::queue_on(ctx, "index value", [&](hipStream_t stream) {
            hipLaunchKernelGGL(hmr::check_value_kernel, dim3(1), dim3(1), 0, stream, base, is64, d, slot);
            return true;
        });
    });
}

hmr_status hmr_index_select(hmr_context_t ctx, const hmr_tensor_desc *out, const hmr_tensor_desc *src,
                            const hmr_tensor_desc *index, int32_t dim, int32_t wrap_negative) {
    return fenced([&] {
        int64_t n = 0, m = 0, count = 0;
        if (hmr_status s = hmr::check_desc(*out, n)) return s;
        if (hmr_status s = hmr::check_desc(*src, m)) return s;
        if (hmr_status s = hmr::check_desc(*index, count)) return s;
        if (dim < 0 || dim >= out->ndim) return fail(HMR_INVALID, "index_select: the dimension is out of range");
        if (hmr_status s = hmr::check_same_sizes(*out, *src, dim)) return s;
        if (index->ndim != 1 || index->sizes[0] != out->sizes[dim]) return fail(HMR_INVALID, "index_select: the index doesn't match the output");
        if (!hmr::is_index_dtype(index->dtype)) return fail(HMR_INVALID, "index_select: unsupported dtype");
        if (n == 0) return HMR_OK;
        const int is64 = index->dtype == HMR_I64;
        const int64_t wrap = wrap_negative ? src->sizes[dim] : 0;
        const int elem = hmr::dtype_size(out->dtype);
        // The index walks along `dim` only.
        hmr_tensor_desc walk = *out;
        for (int k = 0; k < walk.ndim; ++k) walk.strides[k] = k == dim ? index->strides[0] : 0;
        const hmr_tensor_desc *const ops[3] = {out, src, &walk};
        const hmr::Dims d = hmr::dims_of(*out, ops, dim);
        // Rows of whole aligned tiles: the innermost dimension isn't the indexed one and is contiguous in both.
        const int last = out->ndim - 1;
        const int vec = 16 / elem;
        bool rows = last != dim && out->strides[last] == 1 && src->strides[last] == 1 && out->sizes[last] % vec == 0 &&
                    n < (int64_t{1} << 31) && reinterpret_cast<uintptr_t>(hmr::first_of(*out)) % 16 == 0 &&
                    reinterpret_cast<uintptr_t>(hmr::first_of(*src)) % 16 == 0;
        for (int k = 0; rows && k < last; ++k) rows = out->strides[k] % vec == 0 && src->strides[k] % vec == 0;
        return hmr::queue_on(ctx, "index_select", [&](hipStream_t stream) {
            if (src->dtype != out->dtype) return false;
            return hmr::with_word(elem, [&](auto w) {
                using W = typename decltype(w)::type;
                if (rows) {
                    hmr::RowsOfTiles a{};
                    a.out = hmr::first_of(*out);
                    a.src = hmr::first_of(*src);
                    a.index = hmr::first_of(*index);
                    a.is64 = is64;
                    a.wrap = wrap;
                    a.index_stride = index->strides[0];
                    a.tiles_per_row = static_cast<uint32_t>(out->sizes[last] / vec);
                    a.tiles_div = hmr::make_fastdiv(a.tiles_per_row);
                    a.n_tiles = n / vec;
                    a.nouter = 0;
                    a.at = -1;
                    int64_t span = 1;
                    for (int k = 0; k < out->ndim; ++k) span += (out->sizes[k] - 1) * out->strides[k];
                    a.out32 = span * elem <= hmr::kNarrowSpanBytes && n * elem < hmr::kStreamStoreBytes ? 1 : 0;
                    for (int k = last - 1; k >= 0; --k) {
                        if (k == dim) a.at = a.nouter;
                        a.div[a.nouter] = hmr::make_fastdiv(static_cast<uint32_t>(out->sizes[k]));
                        a.stride[0][a.nouter] = out->strides[k];
                        a.stride[1][a.nouter] = src->strides[k];
                        ++a.nouter;
                    }
                    const int64_t per_block = int64_t{4} * hmr::kBlock;
                    hipLaunchKernelGGL((hmr::select_rows_kernel<W>), dim3(static_cast<unsigned>((a.n_tiles + per_block - 1) / per_block)),
                                       dim3(hmr::kBlock), 0, stream, a);
                } else {
                    hipLaunchKernelGGL((hmr::pick_kernel<W>), dim3(hmr::grid_of((n + 3) / 4)), dim3(hmr::kBlock), 0, stream,
                                       reinterpret_cast<W *>(hmr::first_of(*out)), reinterpret_cast<const W *>(hmr::first_of(*src)),
                                       static_cast<const void *>(hmr::first_of(*index)), is64, hmr::squeezed(d), n, wrap);
                }
            });
        });
    });
}

hmr_status hmr_gather(hmr_context_t ctx, const hmr_tensor_desc *out, const hmr_tensor_desc *src, const hmr_tensor_desc *index,
                      int32_t dim) {
    return fenced([&] {
        int64_t n = 0, m = 0, count = 0;
        if (hmr_status s = hmr::check_desc(*out, n)) return s;
        if (hmr_status s = hmr::check_desc(*src, m)) return s;
        if (hmr_status s = hmr::check_desc(*index, count)) return s;
        if (dim < 0 || dim >= out->ndim) return fail(HMR_INVALID, "gather: the dimension is out of range");
        if (hmr_status s = hmr::check_same_sizes(*out, *index, -1)) return s;
        if (src->ndim != out->ndim) return fail(HMR_INVALID, "kernel operands have different sizes");
        if (!hmr::is_index_dtype(index->dtype)) return fail(HMR_INVALID, "gather: unsupported dtype");
        if (n == 0) return HMR_OK;
        const hmr_tensor_desc *const ops[3] = {out, src, index};
        const hmr::Dims d = hmr::dims_of(*out, ops, dim);
        // Lines of the source staged in LDS: the source runs along `dim` with stride 1, a line fits 64 KB, there
        // are enough lines to cover the GPU, and the picks are dense enough that most of a line's 64-byte sectors
        // would be fetched anyway.
        const int elem = hmr::dtype_size(out->dtype);
        const int64_t picks = out->sizes[dim], length = src->sizes[dim], lines = n / picks;
        const bool by_lines = src->strides[dim] == 1 && length * elem <= 65536 && lines >= hmr::kMinLines &&
                              picks * 64 >= length * elem / 2 && picks >= 64;
        return hmr::queue_on(ctx, "gather", [&](hipStream_t stream) {
            if (src->dtype != out->dtype) return false;
            return hmr::with_word(elem, [&](auto w) {
                using W = typename decltype(w)::type;
                if (by_lines) {
                    const unsigned grid = static_cast<unsigned>(lines < (int64_t{1} << 20) ? lines : (int64_t{1} << 20));
                    auto run = [&](auto bytes) {
                        hipLaunchKernelGGL((hmr::gather_lines_kernel<W, decltype(bytes)::value>), dim3(grid), dim3(hmr::kBlock), 0, stream,
                                           reinterpret_cast<W *>(hmr::first_of(*out)), reinterpret_cast<const W *>(hmr::first_of(*src)),
                                           static_cast<const void *>(hmr::first_of(*index)), index->dtype == HMR_I64 ? 1 : 0, d, lines,
                                           picks, length);
                    };
                    if (length * elem <= 8192) run(hmr::IntTag<8192>{});
                    else if (length * elem <= 16384) run(hmr::IntTag<16384>{});
                    else if (length * elem <= 32768) run(hmr::IntTag<32768>{});
                    else run(hmr::IntTag<65536>{});
                    return;
                }
                hipLaunchKernelGGL((hmr::pick_kernel<W>), dim3(hmr::grid_of((n + 3) / 4)), dim3(hmr::kBlock), 0, stream,
                                   reinterpret_cast<W *>(hmr::first_of(*out)), reinterpret_cast<const W *>(hmr::first_of(*src)),
                                   static_cast<const void *>(hmr::first_of(*index)), index->dtype == HMR_I64 ? 1 : 0, hmr::squeezed(d), n,
                                   int64_t{0});
            });
        });
    });
}

hmr_status hmr_index_add_workspace(int64_t m, int64_t size, int64_t *bytes) {
    return fenced([&] {
        if (m < 0 || size < 0) return fail(HMR_INVALID, "index_add_workspace: negative size");
        if (m >= (int64_t{1} << 31) || size >= (int64_t{1} << 32)) {
            return fail(HMR_INVALID, "index_add: more than 2^31 - 1 positions or 2^32 - 1 slices");
        }
        *bytes = m == 0 ? 0 : hmr::sort_layout(m).bytes;
        return HMR_OK;
    });
}

hmr_status hmr_scatter_add_workspace(int64_t n, int64_t *bytes) {
    return fenced([&] {
        if (n < 0) return fail(HMR_INVALID, "scatter_add_workspace: negative size");
        if (n >= (int64_t{1} << 31)) return fail(HMR_INVALID, "scatter_add: more than 2^31 - 1 positions");
        *bytes = n == 0 ? 0 : hmr::sort_layout(n).bytes;
        return HMR_OK;
    });
}

hmr_status hmr_index_add(hmr_context_t ctx, const hmr_tensor_desc *out, const hmr_tensor_desc *src, const hmr_tensor_desc *index,
                         int32_t dim, void *workspace, int64_t workspace_bytes) {
    return fenced([&] {
        int64_t n = 0, total = 0, m = 0;
        if (hmr_status s = hmr::check_desc(*out, n)) return s;
        if (hmr_status s = hmr::check_desc(*src, total)) return s;
        if (hmr_status s = hmr::check_desc(*index, m)) return s;
        if (dim < 0 || dim >= out->ndim) return fail(HMR_INVALID, "index_add: the dimension is out of range");
        if (hmr_status s = hmr::check_same_sizes(*out, *src, dim)) return s;
        if (index->ndim > 1 || m != src->sizes[dim]) return fail(HMR_INVALID, "index_add: the index doesn't match the source");
        if (!hmr::is_index_dtype(index->dtype)) return fail(HMR_INVALID, "index_add: unsupported dtype");
        if (total == 0) return HMR_OK;
        int64_t need = 0;
        if (hmr_status s = hmr_index_add_workspace(m, out->sizes[dim], &need)) return s;
        if (workspace == nullptr || workspace_bytes < need) return fail(HMR_INVALID, "index_add: the workspace is too small");
        // The slice: every dimension but the indexed one.
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
        int lanes = 1;
        while (lanes < hmr::kBlock && lanes < slice) lanes <<= 1;
        uint64_t *words = static_cast<uint64_t *>(workspace);
        const int key_bits = hmr::bits_for(static_cast<uint64_t>(out->sizes[dim] > 0 ? out->sizes[dim] - 1 : 0));
        const int64_t index_stride = index->ndim == 1 ? index->strides[0] : 0;
        return hmr::queue_on(ctx, "index_add", [&](hipStream_t stream) {
            if (src->dtype != out->dtype) return false;
            return hmr::with_any_type(out->dtype, [&](auto t) {
                using T = typename decltype(t)::type;
                hipLaunchKernelGGL(hmr::index_words_kernel, dim3(hmr::grid_of(m)), dim3(hmr::kBlock), 0, stream, words,
                                   static_cast<const void *>(hmr::first_of(*index)), index->dtype == HMR_I64 ? 1 : 0, index_stride, m);
                const uint64_t *sorted = hmr::sort_words(workspace, m, key_bits, stream);
                const int64_t cap = int64_t{1} << 20;
                constexpr int V = 16 / static_cast<int>(sizeof(T));
                T *po = reinterpret_cast<T *>(hmr::first_of(*out));
                const T *ps = reinterpret_cast<const T *>(hmr::first_of(*src));
                // One contiguous run of whole aligned tiles per slice, in both operands?
                const bool tiles = (d.ndim == 0 || (d.ndim == 1 && d.stride[0][0] == 1 && d.stride[1][0] == 1)) && slice % V == 0 &&
                                   reinterpret_cast<uintptr_t>(po) % 16 == 0 && reinterpret_cast<uintptr_t>(ps) % 16 == 0 &&
                                   out->strides[dim] % V == 0 && src->strides[dim] % V == 0;
                if (tiles) {
                    int group = 1;
                    while (group < hmr::kBlock && group < slice / V) group <<= 1;
                    const int64_t groups = (m + hmr::kBlock / group - 1) / (hmr::kBlock / group);
                    hipLaunchKernelGGL((hmr::index_runs_tiles_kernel<T>), dim3(static_cast<unsigned>(groups < cap ? groups : cap)),
                                       dim3(hmr::kBlock), 0, stream, po, ps, sorted, m, slice / V,
                                       out->strides[dim], src->strides[dim], group);
                } else {
                    const int64_t groups = (m + hmr::kBlock / lanes - 1) / (hmr::kBlock / lanes);
                    hipLaunchKernelGGL((hmr::index_runs_kernel<T>), dim3(static_cast<unsigned>(groups < cap ? groups : cap)),
                                       dim3(hmr::kBlock), 0, stream, po, ps, sorted, d, m, slice,
                                       out->strides[dim], src->strides[dim], lanes);
                }
            });
        });
    });
}

hmr_status hmr_scatter_add(hmr_context_t ctx, const hmr_tensor_desc *out, const hmr_tensor_desc *src, const hmr_tensor_desc *index,
                           int32_t dim, void *workspace, int64_t workspace_bytes) {
    return fenced([&] {
        int64_t n = 0, total = 0, count = 0;
        if (hmr_status s = hmr::check_desc(*index, n)) return s;
        if (hmr_status s = hmr::check_desc(*out, total)) return s;
        if (hmr_status s = hmr::check_desc(*src, count)) return s;
        if (dim < 0 || dim >= index->ndim) return fail(HMR_INVALID, "scatter_add: the dimension is out of range");
        if (hmr_status s = hmr::check_same_sizes(*index, *out, dim)) return s;
        if (hmr_status s = hmr::check_same_sizes(*index, *src, -1)) return s;
        if (!hmr::is_index_dtype(index->dtype)) return fail(HMR_INVALID, "scatter_add: unsupported dtype");
        if (n == 0) return HMR_OK;
        int64_t need = 0;
        if (hmr_status s = hmr_scatter_add_workspace(n, &need)) return s;
        if (workspace == nullptr || workspace_bytes < need) return fail(HMR_INVALID, "scatter_add: the workspace is too small");
        if (hmr::reach_of(*out) >= (int64_t{1} << 32) - 1) return fail(HMR_INVALID, "scatter_add: an output of more than 2^32 - 2 elements");
        const hmr_tensor_desc *const ops[3] = {index, out, src};
        const hmr::Dims d = hmr::dims_of(*index, ops, dim);
        uint64_t *words = static_cast<uint64_t *>(workspace);
        const int key_bits = hmr::bits_for(static_cast<uint64_t>(hmr::reach_of(*out)));
        // Line by line in LDS (no global sort, no workspace traffic) when there are enough lines of a size a
        // workgroup takes; one long line, or many tiny ones, go through the global sort.
        const int64_t positions = index->sizes[dim], lines = n / positions, length = out->sizes[dim];
        const int elem = hmr::dtype_size(out->dtype);
        const bool by_lines = lines >= hmr::kMinLines && positions >= 64 && positions <= hmr::kMaxLinePositions &&
                              length * elem <= hmr::kMaxLineBytes && length < (int64_t{1} << 21) && index->strides[dim] == 1 &&
                              src->strides[dim] == 1 && out->strides[dim] == 1;
        return hmr::queue_on(ctx, "scatter_add", [&](hipStream_t stream) {
            if (src->dtype != out->dtype) return false;
            return hmr::with_any_type(out->dtype, [&](auto t) {
                using T = typename decltype(t)::type;
                if (by_lines) {
                    const unsigned grid = static_cast<unsigned>(lines < (int64_t{1} << 20) ? lines : (int64_t{1} << 20));
                    auto run = [&](auto line_bytes, auto padded) {
                        hipLaunchKernelGGL((hmr::scatter_lines_kernel<T, decltype(line_bytes)::value, decltype(padded)::value>),
                                           dim3(grid), dim3(hmr::kBlock), 0, stream, reinterpret_cast<T *>(hmr::first_of(*out)),
                                           reinterpret_cast<const T *>(hmr::first_of(*src)), static_cast<const void *>(hmr::first_of(*index)),
                                           index->dtype == HMR_I64 ? 1 : 0, d, lines, static_cast<int>(positions), static_cast<int>(length));
                    };
                    if (positions <= 512 && length * elem <= 16384) run(hmr::IntTag<16384>{}, hmr::IntTag<512>{});
                    else run(hmr::IntTag<65536>{}, hmr::IntTag<2048>{});
                    return;
                }
                hipLaunchKernelGGL(hmr::scatter_words_kernel, dim3(hmr::grid_of(n)), dim3(hmr::kBlock), 0, stream, words,
                                   static_cast<const void *>(hmr::first_of(*index)), index->dtype == HMR_I64 ? 1 : 0, d, n);
                const uint64_t *sorted = hmr::sort_words(workspace, n, key_bits, stream);
                hipLaunchKernelGGL((hmr::scatter_runs_kernel<T>), dim3(hmr::grid_of(n)), dim3(hmr::kBlock), 0, stream,
                                   reinterpret_cast<T *>(hmr::first_of(*out)), reinterpret_cast<const T *>(hmr::first_of(*src)), sorted, d, n);
            });
        });
    });
}

}  // extern "C"
