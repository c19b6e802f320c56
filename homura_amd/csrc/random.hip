// hmr_random_uniform, hmr_random_normal, hmr_random_int
// (ref: csrc/homura_rocm.h:265-295, csrc/random.hip; the generator is src/ops/random.rs:29-266).
//
// Philox4x32-10 evaluated on the device: block n is the counter [n, n >> 32, 0, 0] under the key
// [seed, seed >> 32]. The caller reserves a call's blocks (from `offset` on) exactly as the CPU
// does, so uniform samples and integers are the CPU's bit for bit; normal samples go through the
// device's f64 log, cos and sin. A thread owns one block: 4 (2 for F64) uniform samples, 2 normal
// samples or 2 integer words, so a wave writes one contiguous span. The kernels only write: they
// are bound by the stores (uniform, integers) or by the f64 transcendentals (normal).
#include <cmath>

#include "mail.hpp"
#include "ew_common.hpp"
#include "normal_math.hpp"

namespace hmr {
namespace {

struct Word4 {
    uint32_t v[4];
};

__device__ __forceinline__ Word4 philox_block(uint64_t n, uint64_t seed) {
    constexpr uint32_t M0 = 0xD2511F53u, M1 = 0xCD9E8D57u, W0 = 0x9E3779B9u, W1 = 0xBB67AE85u;
    uint32_t c0 = static_cast<uint32_t>(n), c1 = static_cast<uint32_t>(n >> 32), c2 = 0, c3 = 0;
    uint32_t k0 = static_cast<uint32_t>(seed), k1 = static_cast<uint32_t>(seed >> 32);
#pragma unroll
    for (int round = 0; round < 10; ++round) {
        if (round > 0) {
            k0 += W0;
            k1 += W1;
        }
        // One 32 x 32 -> 64 multiply each (v_mad_u64_u32) rather than a high and a low half.
        const uint64_t p0 = static_cast<uint64_t>(M0) * c0, p1 = static_cast<uint64_t>(M1) * c2;
        const uint32_t n0 = static_cast<uint32_t>(p1 >> 32) ^ c1 ^ k0, n2 = static_cast<uint32_t>(p0 >> 32) ^ c3 ^ k1;
        c0 = n0, c1 = static_cast<uint32_t>(p1), c2 = n2, c3 = static_cast<uint32_t>(p0);
    }
    return Word4{{c0, c1, c2, c3}};
}

// A uniform f64 in [0, 1) from 53 random bits: (hi * 2^21 + (lo >> 11)) * 2^-53, built from two 32-bit
// conversions; every step is exact. unit_complement is 1 minus it, exact as well (a multiple of 2^-53 in (0, 1]).
__device__ __forceinline__ double unit_f64(uint32_t hi, uint32_t lo) {
    return __builtin_fma(static_cast<double>(lo >> 11), 1.0 / 9007199254740992.0, static_cast<double>(hi) * (1.0 / 4294967296.0));
}
__device__ __forceinline__ double unit_complement(uint32_t hi, uint32_t lo) {
    return __builtin_fma(static_cast<double>(lo >> 11), -1.0 / 9007199254740992.0,
                         __builtin_fma(static_cast<double>(hi), -1.0 / 4294967296.0, 1.0));
}

template <class T>
struct Digits;
template <>
struct Digits<f16_t> {
    static constexpr int value = 11;
};
template <>
struct Digits<bf16_t> {
    static constexpr int value = 8;
};
template <>
struct Digits<float> {
    static constexpr int value = 24;
};

// Stores the first `count` of a thread's PER elements at out + first: one vector store when the
// span is whole and aligned, single elements otherwise (the tail, or an output at an odd offset).
template <class T, int PER>
__device__ __forceinline__ void store_span(T *out, int64_t first, int64_t n, const T (&v)[PER]) {
    T *p = out + first;
    if (first + PER <= n && reinterpret_cast<uintptr_t>(p) % (PER * sizeof(T)) == 0) {
        store_tile<T, PER, false>(reinterpret_cast<char *>(p), v);
    } else {
#pragma unroll
        for (int j = 0; j < PER; ++j) {
            if (first + j < n) p[j] = v[j];
        }
    }
}

// PLAIN (narrow outputs only): `scale` is (to - from) * 2^-bits, exactly, so that bits * scale is the CPU's
// u * (to - from) with u = bits * 2^-bits (scaling by a power of two commutes with the rounding), and the host
// has checked that the largest sample rounds below `to`, so nothing needs mapping back to `from`.
template <class T, bool PLAIN = false>
__global__ void __launch_bounds__(kBlock) uniform_kernel(T *out, int64_t n, int64_t blocks, uint64_t seed, uint64_t offset,
                                                         double from, double to, double scale) {
    constexpr int PER = std::is_same_v<T, double> ? 2 : 4;  // F64 takes two words per value
    const T low = Conv<T>::from_f64(from);
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x; i < blocks;
         i += static_cast<int64_t>(gridDim.x) * kBlock) {
        const Word4 b = philox_block(offset + static_cast<uint64_t>(i), seed);
        T v[PER];
#pragma unroll
        for (int j = 0; j < PER; ++j) {
            double u;
            if constexpr (PLAIN && PER == 4) {
                const double p = static_cast<double>(b.v[j] >> (32 - Digits<T>::value)) * scale;
                v[j] = Conv<T>::from_f64(from + p);
                continue;
            } else if constexpr (PER == 2) {
                u = unit_f64(b.v[2 * j], b.v[2 * j + 1]);
            } else {
                constexpr int bits = Digits<T>::value;
                u = static_cast<double>(b.v[j] >> (32 - bits)) * (1.0 / static_cast<double>(uint64_t{1} << bits));
            }
            const double x = from + u * (to - from);
            T r = Conv<T>::from_f64(x);
            // Rounding can reach the excluded upper bound, which maps to the lower one.
            if (from < to && Conv<T>::to_f64(r) >= to) r = low;
            v[j] = r;
        }
        store_span<T, PER>(out, i * PER, n, v);
    }
}

struct HardwareSeeds {
    static __device__ __forceinline__ double rcp(double x) { return __builtin_amdgcn_rcp(x); }
    static __device__ __forceinline__ double rsq(double x) { return __builtin_amdgcn_rsq(x); }
};

template <class T>
__global__ void __launch_bounds__(kBlock) normal_kernel(T *out, int64_t n, int64_t blocks, uint64_t seed, uint64_t offset,
                                                        double mean, double std) {
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x; i < blocks;
         i += static_cast<int64_t>(gridDim.x) * kBlock) {
        const Word4 b = philox_block(offset + static_cast<uint64_t>(i), seed);
        // Box-Muller in f64: each block gives two normals, the cosine first. Outputs narrower than f64 take
        // the short polynomials of normal_math.hpp.
        const double u1 = unit_complement(b.v[0], b.v[1]), u2 = unit_f64(b.v[2], b.v[3]);
        double r, c, s;
        if constexpr (std::is_same_v<T, double>) {
            const double theta = 2.0 * 3.14159265358979323846 * u2;
            r = sqrt(-2.0 * log(u1)), c = cos(theta), s = sin(theta);
        } else {
            normal_polar<HardwareSeeds>(u1, u2, r, c, s);
        }
        const T v[2] = {Conv<T>::from_f64(mean + std * r * c), Conv<T>::from_f64(mean + std * r * s)};
        store_span<T, 2>(out, 2 * i, n, v);
    }
}

// ---- integers: rejection sampling on 64-bit words -------------------------------------------------
//
// The words of a batch in order are [w0 w1] then [w2 w3] of each block; those >= threshold become
// low + word % range and fill `out` in that order. With threshold 0 nothing is rejected and word j
// is element j. Otherwise the batch is compacted in three launches over tiles of
// HMR_RANDOM_INT_TILE blocks (a workgroup's width): count the accepted words of each group of tiles,
// scan the counts (one workgroup), write each group's accepted words from its offset on, the
// blocks being computed again. The first launch also writes the elements as if nothing were rejected
// and the third returns at once when the total says so, which is the usual case. The workspace holds
// the counts and the offsets (room for one per tile each) and the batch's total (its last word).
static_assert(HMR_RANDOM_INT_TILE == kBlock, "a tile is one workgroup's blocks");

__device__ __forceinline__ void int_words(const Word4 &b, uint64_t (&w)[2]) {
    w[0] = (static_cast<uint64_t>(b.v[0]) << 32) | b.v[1];
    w[1] = (static_cast<uint64_t>(b.v[2]) << 32) | b.v[3];
}

// w % range without a division. A range that rejects nothing divides 2^64, so it is a power of two
// and the remainder is a mask. Otherwise, with magic = floor(2^64 / range), the quotient estimate
// floor(w * magic / 2^64) is the quotient or one less (w / range - w * magic / 2^64 < w / 2^64 < 1),
// so one conditional subtraction finishes; the remainder before it is at most w, which fits.
struct Modulus {
    uint64_t range, magic;
};
inline Modulus make_modulus(uint64_t range) { return Modulus{range, ~uint64_t{0} / range}; }
__device__ __forceinline__ uint64_t remainder(uint64_t w, const Modulus &m) {
    uint64_t r = w - __umul64hi(w, m.magic) * m.range;
    return r >= m.range ? r - m.range : r;
}

__global__ void __launch_bounds__(kBlock) int_all_kernel(int64_t *out, int64_t n, int64_t blocks, uint64_t seed,
                                                         uint64_t offset, int64_t low, uint64_t mask) {
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x; i < blocks;
         i += static_cast<int64_t>(gridDim.x) * kBlock) {
        uint64_t w[2];
        int_words(philox_block(offset + static_cast<uint64_t>(i), seed), w);
        const int64_t v[2] = {static_cast<int64_t>(static_cast<uint64_t>(low) + (w[0] & mask)),
                              static_cast<int64_t>(static_cast<uint64_t>(low) + (w[1] & mask))};
        store_span<int64_t, 2>(out, 2 * i, n, v);
    }
}

// The accepted words of this thread's block (0..2) and, in every thread, the exclusive count of
// accepted words in the threads before it in the workgroup; `total` is the workgroup's count.
__device__ __forceinline__ uint32_t rank_in_tile(uint32_t mine, uint32_t &total) {
    __shared__ uint32_t wave_sum[kBlock / 64];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    uint32_t inclusive = mine;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
        const uint32_t up = static_cast<uint32_t>(__shfl_up(static_cast<int>(inclusive), d, 64));
        if (lane >= d) inclusive += up;
    }
    if (lane == 63) wave_sum[wave] = inclusive;
    __syncthreads();
    uint32_t before = 0;
    total = 0;
#pragma unroll
    for (int k = 0; k < kBlock / 64; ++k) {
        if (k < wave) before += wave_sum[k];
        total += wave_sum[k];
    }
    __syncthreads();  // wave_sum may be written again by the caller's next use
    return before + inclusive - mine;
}

// A workgroup takes kTilesPerGroup tiles one after the other, so that the scan between the two passes
// has few entries (the workspace has room for one per tile; the first `groups` of each half are used).
constexpr int kTilesPerGroup = 64;

// Counts the accepted words of each group and, on the way, writes word j as element j: right as it
// stands when the batch rejects nothing, which is all but certain for a small range (a word is rejected
// with probability range / 2^64 or so). int_write_kernel puts the elements where they belong otherwise.
__global__ void __launch_bounds__(kBlock) int_count_kernel(uint64_t *counts, int64_t *out, int64_t n, int64_t blocks,
                                                           uint64_t seed, uint64_t offset, int64_t low, Modulus modulus,
                                                           uint64_t threshold) {
    uint32_t mine = 0;
    for (int j = 0; j < kTilesPerGroup; ++j) {
        const int64_t i = (static_cast<int64_t>(blockIdx.x) * kTilesPerGroup + j) * kBlock + threadIdx.x;
        if (i < blocks) {
            uint64_t w[2];
            int_words(philox_block(offset + static_cast<uint64_t>(i), seed), w);
            mine += (w[0] >= threshold ? 1u : 0u) + (w[1] >= threshold ? 1u : 0u);
            if (2 * i < n) {
                const int64_t v[2] = {static_cast<int64_t>(static_cast<uint64_t>(low) + remainder(w[0], modulus)),
                                      static_cast<int64_t>(static_cast<uint64_t>(low) + remainder(w[1], modulus))};
                store_span<int64_t, 2>(out, 2 * i, n, v);
            }
        }
    }
    uint32_t total;
    rank_in_tile(mine, total);
    if (threadIdx.x == 0) counts[blockIdx.x] = total;
}

// One workgroup: offsets[t] = the sum of counts[0..t), total = the sum of all. A lane takes `per` adjacent
// counts; the lanes' sums are scanned with shuffles inside a wave and through LDS across the waves.
constexpr int kScanThreads = 1024;
__global__ void __launch_bounds__(kScanThreads) int_scan_kernel(const uint64_t *counts, uint64_t *offsets, uint64_t *total,
                                                                int64_t tiles, uint64_t *mailbox, uint64_t ticket) {
    __shared__ uint64_t wave_sum[kScanThreads / 64];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int64_t per = (tiles + kScanThreads - 1) / kScanThreads;
    const int64_t first = per * threadIdx.x, last = first + per < tiles ? first + per : tiles;
    uint64_t sum = 0;
    for (int64_t t = first; t < last; ++t) sum += counts[t];
    uint64_t x = sum;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
        const uint64_t lo = static_cast<uint32_t>(__shfl_up(static_cast<int>(x), d, 64));
        const uint64_t hi = static_cast<uint32_t>(__shfl_up(static_cast<int>(x >> 32), d, 64));
        if (lane >= d) x += (hi << 32) | lo;
    }
    if (lane == 63) wave_sum[wave] = x;
    __syncthreads();
    uint64_t running = x - sum, all = 0;
#pragma unroll
    for (int w = 0; w < kScanThreads / 64; ++w) {
        running += w < wave ? wave_sum[w] : 0;
        all += wave_sum[w];
    }
    // The batch's count also goes to the mailbox (mail.hpp): the host reads it back at once.
    if (threadIdx.x == 0) {
        *total = all;
        post(mailbox, ticket, all, 0);
    }
    for (int64_t t = first; t < last; ++t) {
        offsets[t] = running;
        running += counts[t];
    }
}

__global__ void __launch_bounds__(kBlock) int_write_kernel(int64_t *out, int64_t n, const uint64_t *offsets, int64_t blocks,
                                                           uint64_t seed, uint64_t offset, int64_t low, Modulus modulus,
                                                           uint64_t threshold, const uint64_t *total_accepted) {
    if (*total_accepted == 2 * static_cast<uint64_t>(blocks)) return;  // nothing rejected: int_count_kernel wrote it all
    uint64_t running = offsets[blockIdx.x];  // accepted words before this group's first tile
    for (int j = 0; j < kTilesPerGroup; ++j) {
        const int64_t i = (static_cast<int64_t>(blockIdx.x) * kTilesPerGroup + j) * kBlock + threadIdx.x;
        uint64_t w[2] = {0, 0};
        bool take[2] = {false, false};
        if (i < blocks) {
            int_words(philox_block(offset + static_cast<uint64_t>(i), seed), w);
            take[0] = w[0] >= threshold;
            take[1] = w[1] >= threshold;
        }
        uint32_t total;
        uint64_t at = running + rank_in_tile((take[0] ? 1u : 0u) + (take[1] ? 1u : 0u), total);
#pragma unroll
        for (int k = 0; k < 2; ++k) {
            if (!take[k]) continue;
            if (at < static_cast<uint64_t>(n)) out[at] = static_cast<int64_t>(static_cast<uint64_t>(low) + remainder(w[k], modulus));
            ++at;
        }
        running += total;
    }
}

// With a cap below the need a thread takes several blocks. The normal samples want that: the constants of
// their arithmetic and the key schedule are then set up once per thread (190 -> 170 us for 67 million f32
// samples). The kernels that mostly write are faster with a workgroup per tile.
constexpr int64_t kNormalGrid = 16384;
inline unsigned grid_of(int64_t threads, int64_t cap = int64_t{1} << 22) {
    const int64_t want = (threads + kBlock - 1) / kBlock;
    return static_cast<unsigned>(want < 1 ? 1 : (want < cap ? want : cap));
}

// The flat contiguous output of a sampling call: its element count and first element.
hmr_status flat_output(const hmr_tensor_desc &out, int64_t &n, char *&first) {
    if (hmr_status s = check_desc(out, n)) return s;
    int64_t expect = 1;
    for (int d = out.ndim - 1; d >= 0; --d) {
        if (out.sizes[d] != 1 && out.strides[d] != expect) return fail(HMR_INVALID, "random sampling writes a contiguous tensor");
        expect *= out.sizes[d];
    }
    first = static_cast<char *>(out.data) + out.offset * dtype_size(out.dtype);
    return HMR_OK;
}

}  // namespace
}  // namespace hmr

extern "C" {

hmr_status hmr_random_uniform(hmr_context_t ctx, const hmr_tensor_desc *out, uint64_t seed, uint64_t offset, double from,
                              double to) {
    return hmr::fenced([&] {
        int64_t n = 0;
        char *first = nullptr;
        if (hmr_status s = hmr::flat_output(*out, n, first)) return s;
        if (n == 0) return HMR_OK;
        return hmr::queue_on(ctx, "random_uniform", [&](hipStream_t stream) {
            return hmr::with_float_type(out->dtype, [&](auto t) {
                using T = typename decltype(t)::type;
                const int64_t per = std::is_same_v<T, double> ? 2 : 4;
                const int64_t blocks = (n + per - 1) / per;
                if constexpr (!std::is_same_v<T, double>) {
                    constexpr int bits = hmr::Digits<T>::value;
                    const double span = to - from, scale = std::ldexp(span, -bits);
                    const double largest = from + static_cast<double>((uint32_t{1} << bits) - 1) * scale;
                    const bool below = hmr::Conv<T>::to_f64(hmr::Conv<T>::from_f64(largest)) < to;
                    if (std::isfinite(span) && std::ldexp(scale, bits) == span && (below || !(from < to))) {
                        hipLaunchKernelGGL((hmr::uniform_kernel<T, true>), dim3(hmr::grid_of(blocks)), dim3(hmr::kBlock), 0, stream,
                                           reinterpret_cast<T *>(first), n, blocks, seed, offset, from, to, scale);
                        return;
                    }
                }
                hipLaunchKernelGGL((hmr::uniform_kernel<T>), dim3(hmr::grid_of(blocks)), dim3(hmr::kBlock), 0, stream,
                                   reinterpret_cast<T *>(first), n, blocks, seed, offset, from, to, 0.0);
            });
        });
    });
}

hmr_status hmr_random_normal(hmr_context_t ctx, const hmr_tensor_desc *out, uint64_t seed, uint64_t offset, double mean,
                             double std) {
    return hmr::fenced([&] {
        int64_t n = 0;
        char *first = nullptr;
        if (hmr_status s = hmr::flat_output(*out, n, first)) return s;
        if (n == 0) return HMR_OK;
        return hmr::queue_on(ctx, "random_normal", [&](hipStream_t stream) {
            return hmr::with_float_type(out->dtype, [&](auto t) {
                using T = typename decltype(t)::type;
                const int64_t blocks = (n + 1) / 2;
                hipLaunchKernelGGL((hmr::normal_kernel<T>), dim3(hmr::grid_of(blocks, hmr::kNormalGrid)), dim3(hmr::kBlock), 0, stream,
                                   reinterpret_cast<T *>(first), n, blocks, seed, offset, mean, std);
            });
        });
    });
}

hmr_status hmr_random_int(hmr_context_t ctx, const hmr_tensor_desc *out, uint64_t seed, uint64_t offset, uint64_t blocks,
                          int64_t low, uint64_t range, uint64_t threshold, void *workspace) {
    return hmr::fenced([&] {
        int64_t n = 0;
        char *first = nullptr;
        if (hmr_status s = hmr::flat_output(*out, n, first)) return s;
        if (out->dtype != HMR_I64) return hmr::fail(HMR_INVALID, "random_int: unsupported dtype");
        if (range == 0) return hmr::fail(HMR_INVALID, "random_int: the range is empty");
        if (blocks > (uint64_t{1} << 62)) return hmr::fail(HMR_INVALID, "random_int: too many blocks");
        if (threshold != 0 && workspace == nullptr) return hmr::fail(HMR_INVALID, "random_int: a workspace is needed to reject words");
        if (threshold == 0 && (range & (range - 1)) != 0) {
            return hmr::fail(HMR_INVALID, "random_int: a range that isn't a power of two rejects words below 2^64 mod range");
        }
        const int64_t nblocks = static_cast<int64_t>(blocks);
        const int64_t tiles = (nblocks + HMR_RANDOM_INT_TILE - 1) / HMR_RANDOM_INT_TILE;
        if (threshold != 0 && tiles > (int64_t{1} << 31) - 1) return hmr::fail(HMR_INVALID, "random_int: too many blocks in one batch");
        if (blocks == 0 && threshold == 0) return HMR_OK;
        if (ctx == nullptr) return hmr::fail(HMR_INVALID, "random_int: null context");
        uint64_t *mailbox = static_cast<uint64_t *>(ctx->mailbox);
        const uint64_t ticket = ++ctx->mail_ticket;
        const hmr_status queued = hmr::queue_on(ctx, "random_int", [&](hipStream_t stream) {
            int64_t *po = reinterpret_cast<int64_t *>(first);
            if (threshold == 0) {
                if (n == 0) return true;
                // Nothing is rejected only when the range divides 2^64: a power of two.
                hipLaunchKernelGGL(hmr::int_all_kernel, dim3(hmr::grid_of(nblocks)), dim3(hmr::kBlock), 0, stream, po, n, nblocks,
                                   seed, offset, low, range - 1);
                return true;
            }
            uint64_t *counts = static_cast<uint64_t *>(workspace), *offsets = counts + tiles, *total = counts + 2 * tiles;
            const int64_t groups = (tiles + hmr::kTilesPerGroup - 1) / hmr::kTilesPerGroup;
            if (groups > 0) {
                hipLaunchKernelGGL(hmr::int_count_kernel, dim3(static_cast<unsigned>(groups)), dim3(hmr::kBlock), 0, stream, counts,
                                   po, n, nblocks, seed, offset, low, hmr::make_modulus(range), threshold);
            }
            hipLaunchKernelGGL(hmr::int_scan_kernel, dim3(1), dim3(hmr::kScanThreads), 0, stream, counts, offsets, total, groups, mailbox, ticket);
            if (groups > 0 && n > 0) {
                hipLaunchKernelGGL(hmr::int_write_kernel, dim3(static_cast<unsigned>(groups)), dim3(hmr::kBlock), 0, stream, po, n,
                                   offsets, nblocks, seed, offset, low, hmr::make_modulus(range), threshold, total);
            }
            return true;
        });
        // A batch that rejects leaves its count in the mailbox as well, for the read-back that follows.
        if (queued == HMR_OK && threshold != 0) {
            const int64_t count_tiles = (static_cast<int64_t>(blocks) + HMR_RANDOM_INT_TILE - 1) / HMR_RANDOM_INT_TILE;
            ctx->mail_src = static_cast<uint64_t *>(workspace) + 2 * count_tiles;
        }
        return queued;
    });
}

}  // extern "C"
