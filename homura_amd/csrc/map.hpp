// The elementwise engine: out[i] = f(in0[i], in1[i], in2[i]) over strided operands.
//
// Replaces the reference's three generic kernels (ref: csrc/elementwise.hip:412-551 and
// csrc/kernel.hpp:83-103, which index every element of every broadcast with int64 div/mod).
// Four kernels, picked on the host from the operands' merged dimensions:
//
//  map_rows_kernel   every operand walks its innermost dimension with stride 1 or 0. A lane owns
//                    V consecutive elements of a row, V = 16 bytes of the widest operand, so the
//                    widest operands move in 128-bit accesses and narrower ones in 64/32/16-bit
//                    accesses, each instruction of a wave covering one contiguous span. The
//                    outer dimensions are resolved once per V elements with 32-bit multiply-shift
//                    division; a contiguous tensor is the one-dimensional case with no division
//                    at all. Stride-0 operands (bias rows, per-row scales, scalars) are read once
//                    per lane-tile and replicated in registers. Each lane runs U tiles per pass,
//                    loads first, stores after, to keep >= 64 bytes per operand in flight.
//  map_tiled_kernel, map_tiled16_kernel
//                    an input (or the output) contiguous along another dimension than the rest: a
//                    transposition. A tile of the two dimensions goes through LDS so that both sides
//                    move whole runs; the 16-byte form serves whole aligned tiles of equal-width
//                    operands, the other one everything else that is long enough to fill a tile.
//  map_any_kernel    anything else (every-other views, misaligned, overflowing 32 bits ...): an
//                    element at a time, four of them per lane in flight, 32-bit multiply-shift
//                    indexing when every offset fits, int64 otherwise.
//
// A functor F describes one op:
//   static constexpr int N;           number of inputs (1..3)
//   using Out, In0, In1, In2;         storage types (unused inputs: hmr::Unused)
//   __device__ Out operator()(In0, In1, In2) const;
// Inputs may also be kernel-argument constants (hmr_binary_constant, hmr_where_constant,
// hmr_fill), which cost no memory traffic.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>
#include <string>

#include "common.hpp"
#include "elem.hpp"

namespace hmr {

constexpr int kBlock = 256;      // 4 waves of 64
// The rows kernel: one wave a workgroup, two tiles a lane. With inputs and results both coming from and going to
// HBM (several buffer sets in rotation), many small workgroups keep more independent streams in flight than
// 256-lane workgroups of four tiles a lane did: a 268 MB x + bias went from 72 to 77 % of the peak rate.
constexpr int kRowsBlock = 64;
constexpr int kRowsTiles = 2;
constexpr int kFastDims = 6;     // merged dimensions the 32-bit kernels take
constexpr int kMaxOperands = 4;  // output + 3 inputs
// The vector kernels mark their 128-bit accesses nontemporal (see load_tile). The hint has to be
// fixed at compile time: a run-time choice between the two forms is merged by the compiler into
// one plain access.
constexpr bool kStreamLoads = true;
constexpr bool kStreamStores = false;
// Outputs from this size on are stored with the nontemporal hint (measured: 537 MB outputs of i64 ops and of the
// f32 softmax gain 3-6 %, 268 MB outputs lose 3-5 %; the memory-side cache holds 256 MB).
constexpr int64_t kStreamStoreBytes = int64_t{384} << 20;
// Calls that move no more than this in all go through the caches (the memory-side cache holds 256 MB).
constexpr int64_t kCacheResidentBytes = int64_t{224} << 20;

struct Unused {};

// ---- host-side view of one call ----------------------------------------------------------------

// The operands of a call after this library's own dimension merge (callers merge too, but the
// contract only promises same sizes). Operand 0 is the output.
struct MapCall {
    int nops = 0;  // operands including the output
    int64_t n = 0;
    int ndim = 0;
    int64_t size[HMR_MAX_DIMS];
    int64_t stride[kMaxOperands][HMR_MAX_DIMS];
    char *ptr[kMaxOperands];         // address of element (0,..,0); nullptr for a constant
    int elem_size[kMaxOperands];
    uint64_t cbits[kMaxOperands];
    bool is_const[kMaxOperands];
    int compute_units = 256;
};

// Validates one description (ref: csrc/kernel.hpp:62-78): dtype and rank in range, no negative
// size or stride. Leaves the element count in n.
hmr_status check_desc(const hmr_tensor_desc &d, int64_t &n, bool negative_strides = false);

// Builds the call for `descs[0..count)` (descs[k] == nullptr marks a constant with bits[k]):
// checks that all have the output's sizes, then drops size-1 dimensions and joins neighbours
// that are contiguous with each other in every operand.
hmr_status prepare_map(MapCall &call, int count, const hmr_tensor_desc *const *descs, const uint64_t *bits,
                       bool negative_inputs = false);

// ---- device-side argument blocks ------------------------------------------------------------------

// x / d for 0 <= x < 2^31 and 1 <= d < 2^31 as (x * mul) >> (32 + shift): round-up method.
struct FastDiv {
    uint32_t div;
    uint32_t mul;
    uint32_t shift;
};

inline FastDiv make_fastdiv(uint32_t d) {
    FastDiv f{d, 0, 0};
    uint32_t s = 0;
    while ((1ull << s) < d) ++s;  // ceil(log2 d)
    uint64_t m = ((1ull << 32) * ((1ull << s) - d)) / d + 1;
    f.mul = static_cast<uint32_t>(m);
    f.shift = s;
    return f;
}

__device__ __forceinline__ uint32_t divide(uint32_t x, const FastDiv &f) {
    // floor(x * (2^32 + mul) / 2^(32 + shift)); t <= x < 2^31, so the sum cannot wrap.
    uint32_t t = __umulhi(x, f.mul);
    return (t + x) >> f.shift;
}

template <int NOPS>
struct RowsArgs {
    char *ptr[NOPS];
    uint64_t cbits[NOPS];
    uint32_t const_mask;   // bit k: operand k is a constant
    uint32_t bcast_mask;   // bit k: operand k has inner stride 0
    uint32_t gather;       // nonzero: 2-byte output tiles of eight lanes leave as one 16-byte store
    uint32_t out32;        // nonzero: every byte offset into the output fits 32 bits
    int64_t n;             // elements
    uint32_t inner;        // size of the innermost dimension
    int32_t nouter;        // outer dimensions (0 for contiguous)
    FastDiv div[kFastDims - 1];            // outer dims, innermost first
    int32_t ostride[NOPS][kFastDims - 1];  // their strides, same order, in elements
    FastDiv inner_div;
};

template <int NOPS, class Idx>
struct AnyArgs {
    char *ptr[NOPS];
    uint64_t cbits[NOPS];
    uint32_t const_mask;
    int32_t ndim;
    int64_t n;
    static constexpr int kDims = std::is_same_v<Idx, uint32_t> ? kFastDims : HMR_MAX_DIMS;
    FastDiv div[std::is_same_v<Idx, uint32_t> ? kFastDims : 1];  // innermost first (32-bit only)
    int64_t size64[std::is_same_v<Idx, uint32_t> ? 1 : HMR_MAX_DIMS];
    std::conditional_t<std::is_same_v<Idx, uint32_t>, int32_t, int64_t> stride[NOPS][kDims];  // innermost first
};

// ---- register tiles ---------------------------------------------------------------------------------

// 128-bit words as a native vector type, which the nontemporal builtins accept.
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// NT marks the access nontemporal ("streaming"). Measured on MI355X with an f32 add over
// 3 x 256 MB: plain 5.77 TB/s; nontemporal loads 6.24 TB/s with cold buffers and 6.9-7.6 TB/s
// when the output buffer is one that was written recently (a chain of ops, or a loop that
// recycles its buffers: the memory-side cache absorbs the plain stores); nontemporal stores as
// well: 6.6 TB/s in every case. Loads stream, stores stay plain.
template <class T, int V, bool NT = false>
__device__ __forceinline__ void load_tile(const char *p, T (&r)[V]) {
    constexpr int bytes = V * static_cast<int>(sizeof(T));
    if constexpr (bytes % 16 == 0) {
#pragma unroll
        for (int i = 0; i < bytes / 16; ++i) {
            const u32x4 *q = reinterpret_cast<const u32x4 *>(p) + i;
            u32x4 w = NT ? __builtin_nontemporal_load(q) : *q;
            __builtin_memcpy(reinterpret_cast<char *>(r) + 16 * i, &w, 16);
        }
    } else if constexpr (bytes == 8) {
        uint2 w = *reinterpret_cast<const uint2 *>(p);
        __builtin_memcpy(r, &w, 8);
    } else if constexpr (bytes == 4) {
        uint32_t w = *reinterpret_cast<const uint32_t *>(p);
        __builtin_memcpy(r, &w, 4);
    } else if constexpr (bytes == 2) {
        uint16_t w = *reinterpret_cast<const uint16_t *>(p);
        __builtin_memcpy(r, &w, 2);
    } else {
        static_assert(bytes == 1, "tile size");
        __builtin_memcpy(r, p, 1);
    }
}

// Where a kernel's 16-byte stores go. They write through the compute die's L2 (scope bits sc0 sc1 on the store):
// an L2 that keeps the dirty lines of a stream writes them back in bursts that the loads wait behind (measured on
// MI355X, a 134 MB -> 134 MB stream whose buffers come from HBM: plain stores 46 us, nontemporal ones 43.7,
// write-through ones 41.7; an f32 add of 3 x 67 MB 31.7 / 31.5 / 29.4 us), and the memory-side cache still keeps the
// result for the next kernel (the same stream reading what the previous launch wrote: 39.3 / 43.5 / 37.2 us). The
// scope bits are reachable through the buffer form of the store only, whose offset has 32 bits: an output that
// spans more (`narrow` false) takes nontemporal global stores.
struct OutStores {
    __amdgpu_buffer_rsrc_t rsrc;
    char *base;
    bool narrow;
    __device__ __forceinline__ OutStores(char *out, bool fits32)
        : rsrc(__builtin_amdgcn_make_buffer_rsrc(out, 0, -1, 0x00020000)), base(out), narrow(fits32) {}
    // Stores `w` at byte offset `at` of the output.
    __device__ __forceinline__ void put16(int64_t at, u32x4 w) const {
        constexpr int kSc0Sc1 = 17;
        if (narrow) __builtin_amdgcn_raw_buffer_store_b128(w, rsrc, static_cast<int>(static_cast<uint32_t>(at)), 0, kSc0Sc1);
        else __builtin_nontemporal_store(w, reinterpret_cast<u32x4 *>(base + at));
    }
};
// The largest span of an output that `OutStores` addresses with 32 bits.
constexpr int64_t kNarrowSpanBytes = (int64_t{1} << 32) - 64;

template <int MODE>
__device__ __forceinline__ void store16(u32x4 *q, u32x4 w) {
    if constexpr (MODE == 1) __builtin_nontemporal_store(w, q);
    else *q = w;
}

template <class T, int V, bool NT = false>
__device__ __forceinline__ void store_tile(char *p, const T (&r)[V]) {
    constexpr int bytes = V * static_cast<int>(sizeof(T));
    if constexpr (bytes % 16 == 0) {
#pragma unroll
        for (int i = 0; i < bytes / 16; ++i) {
            u32x4 w;
            __builtin_memcpy(&w, reinterpret_cast<const char *>(r) + 16 * i, 16);
            u32x4 *q = reinterpret_cast<u32x4 *>(p) + i;
            store16<NT ? 1 : 0>(q, w);
        }
    } else if constexpr (bytes == 8) {
        uint2 w;
        __builtin_memcpy(&w, r, 8);
        *reinterpret_cast<uint2 *>(p) = w;
    } else if constexpr (bytes == 4) {
        uint32_t w;
        __builtin_memcpy(&w, r, 4);
        *reinterpret_cast<uint32_t *>(p) = w;
    } else if constexpr (bytes == 2) {
        uint16_t w;
        __builtin_memcpy(&w, r, 2);
        *reinterpret_cast<uint16_t *>(p) = w;
    } else {
        static_assert(bytes == 1, "tile size");
        __builtin_memcpy(p, r, 1);
    }
}

// A 2-byte tile per lane (a bool mask computed from 8-byte operands) would leave as 2-byte stores, 128 bytes
// per instruction. Eight consecutive lanes hold eight consecutive tiles, so their sixteen bytes are gathered
// into the first of them with data-parallel moves inside the row of 16 lanes and leave as one 16-byte store:
//   pair      lanes 2k:  own bytes + those of lane 2k+1        (quad_perm [1,0,3,2])
//   next_pair lanes 4k:  the pair of lane 4k+2                 (quad_perm [2,3,0,1])
//   far       lanes 8k:  pair and next_pair of lane 8k+4       (row_shl:4)
__device__ __forceinline__ void store_eight_lanes(const OutStores &out, int64_t at, uint16_t own) {
    constexpr int kSwapPairs = 1 | (0 << 2) | (3 << 4) | (2 << 6), kSwapHalves = 2 | (3 << 2) | (0 << 4) | (1 << 6);
    constexpr int kRowShl4 = 0x104;
    const int x = static_cast<int>(own);
    const int pair = x | (__builtin_amdgcn_mov_dpp(x, kSwapPairs, 0xF, 0xF, true) << 16);
    const int next_pair = __builtin_amdgcn_mov_dpp(pair, kSwapHalves, 0xF, 0xF, true);
    const int far0 = __builtin_amdgcn_mov_dpp(pair, kRowShl4, 0xF, 0xF, true);
    const int far1 = __builtin_amdgcn_mov_dpp(next_pair, kRowShl4, 0xF, 0xF, true);
    if ((threadIdx.x & 7u) == 0) {
        u32x4 w = {static_cast<uint32_t>(pair), static_cast<uint32_t>(next_pair), static_cast<uint32_t>(far0),
                   static_cast<uint32_t>(far1)};
        out.put16(at, w);
    }
}

template <class T>
__device__ __forceinline__ T from_cbits(uint64_t bits) {
    if constexpr (std::is_same_v<T, Unused>) {
        return Unused{};
    } else {
        T v;
        __builtin_memcpy(&v, &bits, sizeof(T));
        return v;
    }
}

template <class T>
constexpr int size_or_zero() {
    if constexpr (std::is_same_v<T, Unused>) return 0;
    else return static_cast<int>(sizeof(T));
}

// Bit k of F::kConstantInputs (when a functor has it): input k only ever arrives as a kernel-argument constant.
template <class F, class = void>
struct ConstantInputs {
    static constexpr uint32_t mask = 0;
};
template <class F>
struct ConstantInputs<F, std::void_t<decltype(F::kConstantInputs)>> {
    static constexpr uint32_t mask = F::kConstantInputs;
};

template <class F>
struct MapTraits {
    static constexpr int N = F::N;
    static constexpr uint32_t constant = ConstantInputs<F>::mask;
    static constexpr int so = static_cast<int>(sizeof(typename F::Out));
    // Sizes of the operands that move through memory (0: none, or a constant).
    static constexpr int s0 = (constant & 1u) ? 0 : size_or_zero<typename F::In0>();
    static constexpr int s1 = (constant & 2u) ? 0 : size_or_zero<typename F::In1>();
    static constexpr int s2 = (constant & 4u) ? 0 : size_or_zero<typename F::In2>();
    static constexpr int cmin(int a, int b) { return (b != 0 && b < a) ? b : a; }
    static constexpr int cmax(int a, int b) { return b > a ? b : a; }
    static constexpr int narrow = cmin(cmin(cmin(so, s0), s1), s2);
    static constexpr int wide = cmax(cmax(cmax(so, s0), s1), s2);
    // Elements per lane-tile: 16 bytes of the WIDEST operand, so that no operand needs more than
    // one access per tile and every access instruction of a wave covers one contiguous span
    // (narrower operands move 8, 4 or 2 bytes per lane). Measured on MI355X: letting a lane own
    // 128 contiguous bytes (16 bytes of the narrowest operand) makes each 128-bit load touch 64
    // different cache lines, which with streaming loads multiplies the traffic.
    static constexpr int V = 16 / wide;
    // Tiles per lane per pass.
    static constexpr int U = kRowsTiles;
};

template <class F>
__device__ __forceinline__ typename F::Out apply(const F &f, typename F::In0 a, typename F::In1 b,
                                                 typename F::In2 c) {
    if constexpr (F::N == 1) return f(a);
    else if constexpr (F::N == 2) return f(a, b);
    else return f(a, b, c);
}

// A functor that carries run-time parameters (coefficients in its computation type) takes them from
// the 64-bit constant slots of operands that aren't constants: the output's, then the first input's.
template <class F>
__device__ __forceinline__ F make_functor(const uint64_t *slots) {
    if constexpr (std::is_constructible_v<F, uint64_t, uint64_t>) return F{slots[0], slots[1]};
    else if constexpr (std::is_constructible_v<F, uint64_t>) return F{slots[0]};
    else return F{};
}

// ---- map_rows_kernel ---------------------------------------------------------------------------------
//
// The pass of a workgroup over its U*256 tiles comes in two forms. When every one of those tiles is
// whole (all but the last workgroup of a ragged contiguous tensor) the body is straight-line code:
// every address is computed, every load of every tile is issued, and only then does arithmetic
// start, so a lane has U loads per operand in flight. Operands that are not plain vectors - a
// stride-0 operand or a kernel-argument constant - must not put a branch between those loads (the
// compiler would wait for memory at every join), so they are loaded too, as the aligned 16-byte
// (or narrower) chunk that holds their element, and the element is picked out and replicated
// afterwards. A constant's chunk is read from the output's first bytes and ignored.
// The ragged pass handles partial tiles with per-element accesses.

// The bytes of one operand's tile as they sit in registers between the load and the arithmetic:
// an SSA vector of 32-bit words (never an array in memory, which a variable pick index would pin
// to scratch).
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
template <int BYTES>
struct RawOf;
template <>
struct RawOf<16> {
    using type = u32x4;
};
template <>
struct RawOf<8> {
    using type = u32x2;
};
template <>
struct RawOf<4> {
    using type = uint32_t;
};
template <>
struct RawOf<2> {
    using type = uint16_t;
};
template <>
struct RawOf<1> {
    using type = uint8_t;
};

template <class T, int V>
struct Chunk {
    static constexpr int bytes = V * static_cast<int>(sizeof(T));
    static_assert(bytes == 16 || bytes == 8 || bytes == 4 || bytes == 2 || bytes == 1, "chunk size");
    using Raw = typename RawOf<bytes>::type;
};
template <int V>
struct Chunk<Unused, V> {
    static constexpr int bytes = 0;
    using Raw = Unused;
};

// Loads the chunk at `p` (dense) or the aligned chunk containing the element at `p` (splat);
// `low` is the element's byte offset inside that chunk.
template <class T, int V, bool STREAM = kStreamLoads>
__device__ __forceinline__ typename Chunk<T, V>::Raw load_chunk(const char *p, bool splat, int &low) {
    using Raw = typename Chunk<T, V>::Raw;
    constexpr int bytes = Chunk<T, V>::bytes;
    if constexpr (std::is_same_v<T, Unused>) {
        low = 0;
        return Unused{};
    } else {
    // Pointer arithmetic only: an integer-to-pointer cast would lose the global address space.
    low = static_cast<int>(reinterpret_cast<uintptr_t>(p) & static_cast<uintptr_t>(bytes - 1));
    const Raw *q = reinterpret_cast<const Raw *>(splat ? p - low : p);
    if constexpr (STREAM) return __builtin_nontemporal_load(q);
    else return *q;
    }
}

// The 32-bit word `wi` of a chunk, chosen with selects.
template <class Raw>
__device__ __forceinline__ uint32_t chunk_word(Raw raw, int wi) {
    if constexpr (std::is_same_v<Raw, u32x4>) {
        uint32_t w = raw[0];
        w = wi == 1 ? raw[1] : w;
        w = wi == 2 ? raw[2] : w;
        w = wi == 3 ? raw[3] : w;
        return w;
    } else if constexpr (std::is_same_v<Raw, u32x2>) {
        return wi == 1 ? raw[1] : raw[0];
    } else {
        return static_cast<uint32_t>(raw);
    }
}

// Turns a loaded chunk into the tile's V elements: as loaded (dense), or V copies of the element
// at byte offset `low` (splat), or V copies of the constant.
// L: what was loaded for the input (Unused for an input that is always a constant).
template <class T, class L, int V>
__device__ __forceinline__ void unpack_chunk(typename Chunk<L, V>::Raw raw, bool splat, int low, bool is_const,
                                             uint64_t cbits, T (&r)[V]) {
    if constexpr (std::is_same_v<T, Unused>) {
        return;
    } else if constexpr (std::is_same_v<L, Unused>) {
        const T v = from_cbits<T>(cbits);
#pragma unroll
        for (int i = 0; i < V; ++i) r[i] = v;
    } else {
        if (!splat) {
            __builtin_memcpy(r, &raw, sizeof(raw));
            return;
        }
        uint64_t bits = chunk_word(raw, low >> 2);
        if constexpr (sizeof(T) == 8) bits |= static_cast<uint64_t>(chunk_word(raw, (low >> 2) + 1)) << 32;
        if constexpr (sizeof(T) < 4) bits >>= (low & 3) * 8;
        if (is_const) bits = cbits;
        const T v = from_cbits<T>(bits);
#pragma unroll
        for (int i = 0; i < V; ++i) r[i] = v;
    }
}

// Reads the tile of one input in the ragged pass.
template <class T, int V>
__device__ __forceinline__ void read_ragged(T (&r)[V], const char *base, uint64_t cbits, bool is_const, bool bcast,
                                            int64_t off, int valid) {
    if constexpr (std::is_same_v<T, Unused>) {
        return;
    } else {
        const T *p = reinterpret_cast<const T *>(base + off * static_cast<int64_t>(sizeof(T)));
        if (is_const) {
            T v = from_cbits<T>(cbits);
#pragma unroll
            for (int i = 0; i < V; ++i) r[i] = v;
        } else if (bcast) {
            T v = *p;
#pragma unroll
            for (int i = 0; i < V; ++i) r[i] = v;
        } else {
#pragma unroll
            for (int i = 0; i < V; ++i) {
                if (i < valid) r[i] = p[i];
            }
        }
    }
}

// FLAT: one dimension (contiguous / scalar-broadcast operands); its last tile may be ragged.
// Otherwise the innermost size is a multiple of V and rows never straddle a tile.
// CACHED: bit k set = input k is loaded through the caches (a broadcast operand, read by many waves); the other
// inputs stream past them with nontemporal loads. The choice has to be made at compile time: loads that differ
// only in the hint are folded into one plain load.
template <class F, bool FLAT, int CACHED = 0>
__global__ void __launch_bounds__(kRowsBlock) map_rows_kernel(RowsArgs<F::N + 1> a) {
    using T = MapTraits<F>;
    constexpr int V = T::V, U = T::U, N = F::N;
    using Out = typename F::Out;
    using A = typename F::In0;
    using B = typename F::In1;
    using C = typename F::In2;
    // What is loaded for an input: nothing for one that is always a constant.
    using LA = std::conditional_t<(T::constant & 1u) != 0, Unused, A>;
    using LB = std::conditional_t<(T::constant & 2u) != 0, Unused, B>;
    using LC = std::conditional_t<(T::constant & 4u) != 0, Unused, C>;
    using Off = std::conditional_t<FLAT, int64_t, uint32_t>;
    const F f = make_functor<F>(a.cbits);
    const OutStores out(a.ptr[0], a.out32 != 0);
    const int64_t tiles = (a.n + V - 1) / V;
    const int64_t whole = a.n / V;  // tiles [0, whole) have all V elements
    const bool c0 = a.const_mask & 2u, c1 = a.const_mask & 4u, c2 = a.const_mask & 8u;
    // "splat": the operand contributes one element per tile (stride 0 inside the tile, or a constant).
    const bool s0 = (a.bcast_mask | a.const_mask) & 2u, s1 = (a.bcast_mask | a.const_mask) & 4u,
               s2 = (a.bcast_mask | a.const_mask) & 8u;
    for (int64_t base = static_cast<int64_t>(blockIdx.x) * (U * kRowsBlock); base < tiles;
         base += static_cast<int64_t>(gridDim.x) * (U * kRowsBlock)) {
        const int64_t t0 = base + threadIdx.x;
        // Element offsets of tile t in each operand.
        auto offsets = [&](int64_t t, Off(&off)[4]) {
            if constexpr (FLAT) {
                const int64_t e = t * V;
                off[0] = e;
                off[1] = s0 ? 0 : e;
                off[2] = s1 ? 0 : e;
                off[3] = s2 ? 0 : e;
            } else {
                const uint32_t e32 = static_cast<uint32_t>(t * V);
                uint32_t row = divide(e32, a.inner_div);
                const uint32_t col = e32 - row * a.inner;
                off[0] = col;
                off[1] = s0 ? 0 : col;
                off[2] = s1 ? 0 : col;
                off[3] = s2 ? 0 : col;
                for (int d = 0; d < a.nouter; ++d) {
                    const uint32_t q = divide(row, a.div[d]);
                    const uint32_t idx = row - q * a.div[d].div;
                    row = q;
                    off[0] += idx * static_cast<uint32_t>(a.ostride[0][d]);
                    if constexpr (N >= 1) off[1] += idx * static_cast<uint32_t>(a.ostride[1][d]);
                    if constexpr (N >= 2) off[2] += idx * static_cast<uint32_t>(a.ostride[2][d]);
                    if constexpr (N >= 3) off[3] += idx * static_cast<uint32_t>(a.ostride[3][d]);
                }
            }
        };
        if (base + U * kRowsBlock <= whole) {
            // Whole pass: addresses, then all loads, then arithmetic and stores.
            typename Chunk<LA, V>::Raw wa[U];
            typename Chunk<LB, V>::Raw wb[U];
            typename Chunk<LC, V>::Raw wc[U];
            int la[U], lb[U], lc[U];
            Off oo[U];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                Off off[4];
                offsets(t0 + static_cast<int64_t>(u) * kRowsBlock, off);
                oo[u] = off[0];
                wa[u] = load_chunk<LA, V, kStreamLoads && !(CACHED & 1)>(a.ptr[1] + static_cast<int64_t>(off[1]) * static_cast<int64_t>(sizeof(A)), s0, la[u]);
                if constexpr (N >= 2) {
                    wb[u] = load_chunk<LB, V, kStreamLoads && !(CACHED & 2)>(a.ptr[2] + static_cast<int64_t>(off[2]) * static_cast<int64_t>(sizeof(B)), s1, lb[u]);
                }
                if constexpr (N >= 3) {
                    wc[u] = load_chunk<LC, V, kStreamLoads && !(CACHED & 4)>(a.ptr[3] + static_cast<int64_t>(off[3]) * static_cast<int64_t>(sizeof(C)), s2, lc[u]);
                }
            }
#pragma unroll
            for (int u = 0; u < U; ++u) {
                A ra[V];
                B rb[V];
                C rc[V];
                unpack_chunk<A, LA, V>(wa[u], s0, la[u], c0, a.cbits[1], ra);
                if constexpr (N >= 2) unpack_chunk<B, LB, V>(wb[u], s1, lb[u], c1, a.cbits[2], rb);
                if constexpr (N >= 3) unpack_chunk<C, LC, V>(wc[u], s2, lc[u], c2, a.cbits[3], rc);
                Out ro[V];
#pragma unroll
                for (int i = 0; i < V; ++i) ro[i] = apply(f, ra[i], rb[i], rc[i]);
                const int64_t at = static_cast<int64_t>(oo[u]) * static_cast<int64_t>(sizeof(Out));
                if constexpr (V * sizeof(Out) == 2) {
                    if (a.gather) {
                        uint16_t w;
                        __builtin_memcpy(&w, ro, 2);
                        store_eight_lanes(out, at, w);
                        continue;
                    }
                }
                if constexpr (V * sizeof(Out) == 16) {
                    u32x4 w;
                    __builtin_memcpy(&w, ro, 16);
                    out.put16(at, w);
                } else {
                    store_tile<Out, V, false>(a.ptr[0] + at, ro);
                }
            }
        } else {
            // Ragged pass (the last workgroup): tile by tile, partial tiles element by element.
            for (int u = 0; u < U; ++u) {
                const int64_t t = t0 + static_cast<int64_t>(u) * kRowsBlock;
                if (t >= tiles) break;
                const int64_t rem = a.n - t * V;
                const int valid = rem >= V ? V : static_cast<int>(rem);
                Off off[4];
                offsets(t, off);
                A xa[V];
                B xb[V];
                C xc[V];
                read_ragged<A, V>(xa, a.ptr[1], a.cbits[1], c0, s0, off[1], valid);
                if constexpr (N >= 2) read_ragged<B, V>(xb, a.ptr[2], a.cbits[2], c1, s1, off[2], valid);
                if constexpr (N >= 3) read_ragged<C, V>(xc, a.ptr[3], a.cbits[3], c2, s2, off[3], valid);
                Out *po = reinterpret_cast<Out *>(a.ptr[0] + static_cast<int64_t>(off[0]) * static_cast<int64_t>(sizeof(Out)));
#pragma unroll
                for (int i = 0; i < V; ++i) {
                    if (i < valid) po[i] = apply(f, xa[i], xb[i], xc[i]);
                }
            }
        }
    }
}

template <class T, class Idx>
__device__ __forceinline__ T read_one(const char *base, uint64_t cbits, bool is_const, Idx off) {
    if constexpr (std::is_same_v<T, Unused>) {
        return Unused{};
    } else {
        if (is_const) return from_cbits<T>(cbits);
        return *reinterpret_cast<const T *>(base + static_cast<int64_t>(off) * static_cast<int64_t>(sizeof(T)));
    }
}

// Elements per lane and pass of the general kernel: four with 32-bit offsets, one with 64-bit ones (whose
// divisions are the cost there).
template <class Idx>
constexpr int kAnyPerLane = std::is_same_v<Idx, uint32_t> ? 4 : 1;

template <class F, class Idx>
__global__ void __launch_bounds__(kBlock) map_any_kernel(AnyArgs<F::N + 1, Idx> a) {
    constexpr int N = F::N;
    using Out = typename F::Out;
    const F f = make_functor<F>(a.cbits);
    const bool c0 = a.const_mask & 2u, c1 = a.const_mask & 4u, c2 = a.const_mask & 8u;
    // Signed: an input's strides may be negative (hmr_flip); every partial sum fits 31 bits then.
    using Off = std::conditional_t<std::is_same_v<Idx, uint32_t>, int32_t, int64_t>;
    // Several elements per lane, a workgroup apart, every load issued before the first store: with one element
    // per lane a wave has a single load in flight, and a strided view (every other column of an f32 matrix) ran
    // at 88 us where the lines it touches take 62 at the memory's rate.
    constexpr int U = kAnyPerLane<Idx>;
    for (int64_t base = static_cast<int64_t>(blockIdx.x) * (U * kBlock); base < a.n;
         base += static_cast<int64_t>(gridDim.x) * (U * kBlock)) {
        Off out_off[U];
        bool valid[U];
        typename F::In0 x[U];
        typename F::In1 y[U];
        typename F::In2 z[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int64_t wanted = base + static_cast<int64_t>(u) * kBlock + threadIdx.x;
            valid[u] = wanted < a.n;
            const int64_t i = valid[u] ? wanted : a.n - 1;  // past the end: the last element again, not stored
            Off off[4] = {0, 0, 0, 0};
            if constexpr (std::is_same_v<Idx, uint32_t>) {
                uint32_t rest = static_cast<uint32_t>(i);
                for (int d = 0; d < a.ndim; ++d) {
                    uint32_t q = divide(rest, a.div[d]);
                    uint32_t idx = rest - q * a.div[d].div;
                    rest = q;
#pragma unroll
                    for (int k = 0; k <= N; ++k) off[k] += static_cast<int32_t>(idx) * a.stride[k][d];
                }
            } else {
                int64_t rest = i;
                for (int d = 0; d < a.ndim; ++d) {
                    int64_t q = rest / a.size64[d];
                    int64_t idx = rest - q * a.size64[d];
                    rest = q;
#pragma unroll
                    for (int k = 0; k <= N; ++k) off[k] += idx * a.stride[k][d];
                }
            }
            out_off[u] = off[0];
            x[u] = read_one<typename F::In0, Off>(a.ptr[1], a.cbits[1], c0, off[1]);
            if constexpr (N >= 2) y[u] = read_one<typename F::In1, Off>(a.ptr[2], a.cbits[2], c1, off[2]);
            if constexpr (N >= 3) z[u] = read_one<typename F::In2, Off>(a.ptr[3], a.cbits[3], c2, off[3]);
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const Out r = apply(f, x[u], y[u], z[u]);
            if (valid[u]) {
                *reinterpret_cast<Out *>(a.ptr[0] + static_cast<int64_t>(out_off[u]) * static_cast<int64_t>(sizeof(Out))) = r;
            }
        }
    }
}

// ---- map_tiled_kernel ---------------------------------------------------------------------------------
//
// A transposed operand: the output runs along its innermost dimension `a` while an input is contiguous along
// another dimension `b` (a transposed or permuted view made contiguous, or combined with operands that are not
// transposed). One element per lane in the general kernel leaves that input's wave-wide loads 64 separate
// sectors (a transposed f32 [8192, 8192] copy: 321 us, 21 % of the memory's rate). Here a workgroup takes a
// tile of S x S elements of the (a, b) plane: every transposed input's tile is read with the lanes along `b` -
// runs of 256 bytes - and parked in LDS; then the lanes turn to run along `a`, read the parked tiles across,
// read the inputs that are not transposed directly, and store the output in runs of 256 bytes.
// A lane moves P consecutive elements (4 bytes of the widest operand, at most two), so S = 64 P.

template <class F>
struct TiledTraits {
    static constexpr int wide = MapTraits<F>::wide;
    static constexpr int P = wide >= 4 ? 1 : 2;
    static constexpr int S = 64 * P;
    static constexpr int kPad = 1;
    // LDS for the tiles of all inputs (each could be the transposed one).
    static constexpr int lds_bytes = S * (S + kPad) * (MapTraits<F>::s0 + MapTraits<F>::s1 + MapTraits<F>::s2);
};

template <int NOPS>
struct TiledArgs {
    char *ptr[NOPS];
    uint64_t cbits[NOPS];
    uint32_t const_mask;  // bit k: operand k is a constant
    uint32_t turned_mask;  // bit k: input k is contiguous along b and goes through LDS
    uint32_t size_a, size_b;
    int32_t stride_a[NOPS], stride_b[NOPS];  // in elements
    FastDiv tiles_a, tiles_b;                // tiles along a, then along b, then the outer dimensions
    int32_t nouter;
    FastDiv div[kFastDims - 2];
    int32_t ostride[NOPS][kFastDims - 2];
};

// The tile of a workgroup and the element offsets of its outer coordinates. Which tiles run at the same time
// decides what the memory sees. Numbered along one dimension, the tiles in flight differ in one coordinate only,
// and with a power-of-two pitch their pieces lie a multiple of that pitch apart, on few memory channels: an f32
// [8192, 8192] transposition took 115-131 us in either plain order. Two orders avoid that:
//   BAND == 0  the tile along `b` is shifted by the one along `a` (a diagonal): 92 us for that kernel. The pieces in
//              flight are scattered one per row, which suits the shorter runs of 1- and 2-byte elements.
//   BAND > 0   bands of BAND tiles along `b`; within a band along `b` first (shifted as above), then along `a`: the
//              512 workgroups in flight cover 64 x 8 tiles, kilobytes of every row they touch on both sides. For
//              4- and 8-byte elements (512-byte runs) this is 3 % slower on f32 [8192, 8192] and 23-24 % faster on
//              [8320, 8064], [32768, 2048] and i64 [8320, 8064], within 4 % elsewhere.
template <int N, int BAND, class Args>
__device__ __forceinline__ void which_tile(const Args &a, uint32_t &ta, uint32_t &tb, int64_t (&base)[4]) {
    uint32_t rest = blockIdx.x;
    uint32_t q = divide(rest, a.tiles_a);
    ta = rest - q * a.tiles_a.div;
    rest = q;
    q = divide(rest, a.tiles_b);
    if constexpr (BAND > 0) {
        const uint32_t t = (rest - q * a.tiles_b.div) * a.tiles_a.div + ta;  // the tile's number in its plane
        const uint32_t per_band = BAND * a.tiles_a.div;
        const uint32_t band = t / per_band, within = t - band * per_band;
        const uint32_t start = band * BAND;
        const uint32_t width = a.tiles_b.div - start < BAND ? a.tiles_b.div - start : BAND;  // the last band may be narrower
        ta = within / width;
        tb = start + (within - ta * width + ta) % width;
    } else {
        const uint32_t shifted = rest - q * a.tiles_b.div + ta;
        tb = shifted - divide(shifted, a.tiles_b) * a.tiles_b.div;
    }
    rest = q;
    for (int d = 0; d < a.nouter; ++d) {
        q = divide(rest, a.div[d]);
        const int64_t idx = rest - q * a.div[d].div;
        rest = q;
#pragma unroll
        for (int k = 0; k <= N; ++k) base[k] += idx * a.ostride[k][d];
    }
}

template <class T, int S, int PAD>
struct TileOf {
    T cell[S][S + PAD];
};
template <int S, int PAD>
struct TileOf<Unused, S, PAD> {};

template <class F>
__global__ void __launch_bounds__(kBlock) map_tiled_kernel(TiledArgs<F::N + 1> a) {
    using TT = TiledTraits<F>;
    constexpr int N = F::N, P = TT::P, S = TT::S, PAD = TT::kPad;
    using Out = typename F::Out;
    using A = typename F::In0;
    using B = typename F::In1;
    using C = typename F::In2;
    __shared__ TileOf<A, S, PAD> tile_a;
    __shared__ TileOf<B, S, PAD> tile_b;
    __shared__ TileOf<C, S, PAD> tile_c;
    const F f = make_functor<F>(a.cbits);
    const int wave = threadIdx.x / 64, lane = threadIdx.x % 64;
    uint32_t ta, tb;
    int64_t base[4] = {0, 0, 0, 0};
    which_tile<N, 0>(a, ta, tb, base);
    const uint32_t a0 = ta * S, b0 = tb * S;
    // Phase 1: the turned inputs, lanes along b.
    auto park = [&](auto &tile, int k, auto zero) {
        using T = decltype(zero);
        if (!((a.turned_mask >> k) & 1u)) return;
        const T *src = reinterpret_cast<const T *>(a.ptr[k]) + base[k];
        const uint32_t bb = b0 + lane * P;
        constexpr int kAhead = 8;  // rows requested before the first is parked
        for (int r0 = wave; r0 < S; r0 += 4 * kAhead) {
            T v[kAhead][P];
#pragma unroll
            for (int u = 0; u < kAhead; ++u) {
                const uint32_t aa = a0 + r0 + 4 * u;
#pragma unroll
                for (int p = 0; p < P; ++p) {
                    const bool in = aa < a.size_a && bb + p < a.size_b && r0 + 4 * u < S;
                    v[u][p] = in ? src[static_cast<int64_t>(aa) * a.stride_a[k] + (bb + p)] : T{};
                }
            }
#pragma unroll
            for (int u = 0; u < kAhead; ++u) {
                if (r0 + 4 * u < S) {
#pragma unroll
                    for (int p = 0; p < P; ++p) tile.cell[r0 + 4 * u][lane * P + p] = v[u][p];
                }
            }
        }
    };
    park(tile_a, 1, A{});
    if constexpr (N >= 2) park(tile_b, 2, B{});
    if constexpr (N >= 3) park(tile_c, 3, C{});
    __syncthreads();
    // Phase 2: lanes along a.
    const bool c0 = a.const_mask & 2u, c1 = a.const_mask & 4u, c2 = a.const_mask & 8u;
    auto fetch = [&](auto &tile, int k, bool is_const, uint32_t aa, uint32_t bb, int p, auto zero) {
        using T = decltype(zero);
        if constexpr (std::is_same_v<T, Unused>) {
            return Unused{};
        } else {
            if (is_const) return from_cbits<T>(a.cbits[k]);
            if ((a.turned_mask >> k) & 1u) return tile.cell[aa - a0][bb - b0];
            (void)p;
            return reinterpret_cast<const T *>(a.ptr[k])[base[k] + static_cast<int64_t>(aa) * a.stride_a[k] +
                                                        static_cast<int64_t>(bb) * a.stride_b[k]];
        }
    };
    Out *out = reinterpret_cast<Out *>(a.ptr[0]) + base[0];
    for (int r = wave; r < S; r += 4) {
        const uint32_t bb = b0 + r;
        if (bb >= a.size_b) break;
#pragma unroll
        for (int p = 0; p < P; ++p) {
            const uint32_t aa = a0 + lane * P + p;
            if (aa < a.size_a) {
                const A x = fetch(tile_a, 1, c0, aa, bb, p, A{});
                const B y = fetch(tile_b, 2, c1, aa, bb, p, B{});
                const C z = fetch(tile_c, 3, c2, aa, bb, p, C{});
                out[static_cast<int64_t>(aa) * a.stride_a[0] + static_cast<int64_t>(bb) * a.stride_b[0]] = apply(f, x, y, z);
            }
        }
    }
}

// The same transposition with 16-byte accesses on both sides, for aligned operands that all have the output's
// element size, exactly one input turned and both dimensions a multiple of 16 bytes. A tile is TA x TB elements; it lies in LDS as the
// turned input has it, rows along `a` of 16-byte slots along `b`, slot s of row r at s ^ (r / V): the 16-byte
// writes of phase 1 spread over all banks, and so do the element reads of phase 2, whose lanes take V
// consecutive rows each at one column. 512 lanes; all loads of a phase are issued before their first use.
template <class F>
struct Tiled16Traits {
    using M = MapTraits<F>;
    static constexpr bool applies = F::N >= 1 && F::N <= 2 && M::s0 == M::so && (F::N == 1 || M::s1 == M::so);
    static constexpr int E = M::so;
    static constexpr int V = 16 / E;
    // Tile edges in elements along a (the output's runs) and along b (the turned input's runs): 64 KiB of
    // 512-byte runs for 4-byte elements, 512- and 256-byte runs for 2-byte ones (measured on bf16
    // [16384, 16384]: 128 x 128 5.5 TB/s, 128 x 256 5.8, 256 x 128 6.1), 256-byte runs for single bytes.
    static constexpr int TA = E == 8 ? 64 : (E == 4 ? 128 : 256);
    static constexpr int TB = E == 8 ? 64 : (E == 1 ? 256 : 128);
    static constexpr int kSlots = TB / V;  // 16-byte slots per row of the tile in LDS
    static constexpr int kLanesA = TA / V;  // lanes along a row of the output
    static constexpr int kThreads = 512;
    static constexpr int kRows1 = kThreads / kSlots, kPasses1 = TA / kRows1;   // phase 1: rows along a
    static constexpr int kRows2 = kThreads / kLanesA, kPasses2 = TB / kRows2;  // phase 2: rows along b
};

template <class F, bool NT>
__global__ void __launch_bounds__(Tiled16Traits<F>::kThreads) map_tiled16_kernel(TiledArgs<F::N + 1> a) {
    using TT = Tiled16Traits<F>;
    constexpr int N = F::N, E = TT::E, V = TT::V, TA = TT::TA, TB = TT::TB, kSlots = TT::kSlots;
    using Out = typename F::Out;
    using A = typename F::In0;
    using B = std::conditional_t<N >= 2, typename F::In1, Unused>;
    __shared__ u32x4 tile[TA * kSlots];
    const F f = make_functor<F>(a.cbits);
    uint32_t ta, tb;
    int64_t base[4] = {0, 0, 0, 0};
    which_tile<N, (E >= 4 ? 8 : 0)>(a, ta, tb, base);
    const uint32_t a0 = ta * TA, b0 = tb * TB;
    const int turned = (a.turned_mask & 2u) ? 1 : 2;
    {
        constexpr int kRows = TT::kRows1, kPasses = TT::kPasses1;
        const int row = threadIdx.x / kSlots, slot = threadIdx.x % kSlots;
        // The last tiles along either dimension may reach past the tensor, by whole 16-byte slots: those slots
        // load the tensor's last row or last slot again (no branch around a load, whose join would wait for it)
        // and are not stored.
        const uint32_t bb = b0 + slot * V < a.size_b ? b0 + slot * V : a.size_b - V;
        const char *src = a.ptr[turned] + (base[turned] + bb) * E;
        u32x4 v[kPasses];
#pragma unroll
        for (int j = 0; j < kPasses; ++j) {
            const uint32_t aa = a0 + j * kRows + row < a.size_a ? a0 + j * kRows + row : a.size_a - 1;
            const u32x4 *p = reinterpret_cast<const u32x4 *>(src + static_cast<int64_t>(aa) * a.stride_a[turned] * E);
            v[j] = NT ? __builtin_nontemporal_load(p) : *p;
        }
#pragma unroll
        for (int j = 0; j < kPasses; ++j) {
            const int r = j * kRows + row;
            tile[r * kSlots + (slot ^ ((r / V) & (kSlots - 1)))] = v[j];
        }
    }
    __syncthreads();
    // Phase 2: rows along b, `lane_a` along a.
    constexpr int kRows = TT::kRows2, kPasses = TT::kPasses2;
    const int row = threadIdx.x / TT::kLanesA, lane_a = threadIdx.x % TT::kLanesA;
    const char *cells = reinterpret_cast<const char *>(tile);
    auto straight = [&](int k, int j, auto zero, auto &r) {
        using X = decltype(zero);
        if constexpr (!std::is_same_v<X, Unused>) {
            if ((a.const_mask >> k) & 1u) {
#pragma unroll
                for (int i = 0; i < V; ++i) r[i] = from_cbits<X>(a.cbits[k]);
            } else if (k != turned) {
                const uint32_t bb = b0 + j * kRows + row < a.size_b ? b0 + j * kRows + row : a.size_b - 1;
                const uint32_t aa = a0 + lane_a * V < a.size_a ? a0 + lane_a * V : a.size_a - V;
                const char *p = a.ptr[k] + (base[k] + static_cast<int64_t>(bb) * a.stride_b[k] + aa) * E;
                load_tile<X, V, NT>(p, r);
            }
        }
    };
    auto parked = [&](int k, int j, auto zero, auto &r) {
        using X = decltype(zero);
        if constexpr (!std::is_same_v<X, Unused>) {
            if (k == turned) {
                const int bl = j * kRows + row;
                const int at = ((bl / V) ^ (lane_a & (kSlots - 1))) * V + bl % V;
#pragma unroll
                for (int i = 0; i < V; ++i) __builtin_memcpy(&r[i], cells + (static_cast<size_t>(lane_a * V + i) * TB + at) * E, E);
            }
        }
    };
    std::conditional_t<std::is_same_v<A, Unused>, char, A> xa[kPasses][V];
    std::conditional_t<std::is_same_v<B, Unused>, char, B> xb[kPasses][V];
#pragma unroll
    for (int j = 0; j < kPasses; ++j) {
        straight(1, j, A{}, xa[j]);
        if constexpr (N >= 2) straight(2, j, B{}, xb[j]);
    }
#pragma unroll
    for (int j = 0; j < kPasses; ++j) {
        parked(1, j, A{}, xa[j]);
        if constexpr (N >= 2) parked(2, j, B{}, xb[j]);
        Out ro[V];
#pragma unroll
        for (int i = 0; i < V; ++i) {
            if constexpr (N >= 2) ro[i] = f(xa[j][i], xb[j][i]);
            else ro[i] = f(xa[j][i]);
        }
        char *po = a.ptr[0] + (base[0] + static_cast<int64_t>(b0 + j * kRows + row) * a.stride_b[0] + a0 + lane_a * V) * E;
        if (b0 + j * kRows + row < a.size_b && a0 + lane_a * V < a.size_a) store_tile<Out, V, NT>(po, ro);
    }
}

// ---- host-side launch -----------------------------------------------------------------------------

inline unsigned grid_for(int64_t work_items, int64_t per_block) {
    int64_t blocks = work_items / per_block + (work_items % per_block != 0);
    const int64_t cap = int64_t{1} << 22;
    if (blocks < 1) blocks = 1;
    return static_cast<unsigned>(blocks < cap ? blocks : cap);
}

// Largest element offset (exclusive bound - 1) operand k can reach.
inline bool fits_32(const MapCall &c) {
    if (c.n >= (int64_t{1} << 31)) return false;
    for (int k = 0; k < c.nops; ++k) {
        if (c.is_const[k]) continue;
        __int128 reach = 0;  // largest magnitude any partial sum of index * stride can take
        for (int d = 0; d < c.ndim; ++d) {
            const __int128 span = static_cast<__int128>(c.size[d] - 1) * c.stride[k][d];
            reach += span < 0 ? -span : span;
        }
        if (reach >= (int64_t{1} << 31)) return false;
    }
    return true;
}

// Which kernel a call takes: 0 contiguous rows kernel, 1 rows kernel with outer dims, 2 any/32, 3 any/64.
template <class F>
int pick_variant(const MapCall &c) {
    using T = MapTraits<F>;
    constexpr int sizes[4] = {T::so, T::s0, T::s1, T::s2};
    // An input the functor declares constant, given as a tensor: only the general kernels read it as one.
    for (int k = 1; k < c.nops; ++k) {
        if (((T::constant >> (k - 1)) & 1u) && !c.is_const[k]) return c.ndim <= kFastDims && fits_32(c) ? 2 : 3;
    }
    // A reversed dimension (negative input stride, hmr_flip only) goes through the general kernels.
    for (int k = 1; k < c.nops; ++k) {
        for (int d = 0; d < c.ndim && !c.is_const[k]; ++d) {
            if (c.stride[k][d] < 0) return c.ndim <= kFastDims && fits_32(c) ? 2 : 3;
        }
    }
    if (c.ndim > kFastDims || !fits_32(c)) return c.ndim <= 1 && c.n < (int64_t{1} << 62) ? -1 : 3;
    if (c.ndim == 0) return 0;
    const int last = c.ndim - 1;
    bool rows = c.stride[0][last] == 1;
    for (int k = 1; rows && k < c.nops; ++k) {
        if (c.is_const[k]) continue;
        rows = c.stride[k][last] == 1 || c.stride[k][last] == 0;
    }
    if (rows) {
        // Every vector access must be aligned: base pointers and (for outer dims) row starts.
        bool aligned = true;
        for (int k = 0; aligned && k < c.nops; ++k) {
            if (c.is_const[k] || c.stride[k][last] == 0) continue;
            int chunk = T::V * sizes[k] < 16 ? T::V * sizes[k] : 16;
            aligned = reinterpret_cast<uintptr_t>(c.ptr[k]) % chunk == 0;
            for (int d = 0; aligned && d < last; ++d) {
                aligned = (c.stride[k][d] * sizes[k]) % chunk == 0;
            }
        }
        if (aligned && c.ndim == 1) return 0;
        if (aligned && c.size[last] % T::V == 0) return 1;
    }
    return 2;
}

// The variant a call takes with -1 (one huge contiguous dimension) resolved to 0 or 3.
template <class F>
int resolve_variant(const MapCall &c) {
    using T = MapTraits<F>;
    int variant = pick_variant<F>(c);
    if (variant == -1) {
        // One huge contiguous dimension (>= 2^31 elements): the FLAT rows kernel indexes in 64 bits.
        bool ok = c.ndim == 0 || c.stride[0][0] == 1;
        for (int k = 1; ok && k < c.nops; ++k) ok = c.is_const[k] || c.stride[k][0] == 1 || c.stride[k][0] == 0;
        constexpr int sizes[4] = {T::so, T::s0, T::s1, T::s2};
        for (int k = 0; ok && k < c.nops; ++k) {
            if (c.is_const[k] || (c.ndim == 1 && c.stride[k][0] == 0)) continue;
            int chunk = T::V * sizes[k] < 16 ? T::V * sizes[k] : 16;
            ok = reinterpret_cast<uintptr_t>(c.ptr[k]) % chunk == 0;
        }
        variant = ok ? 0 : 3;
    }
    return variant;
}

// Kernel arguments of the rows kernel for a call of variant 0 (flat) or 1 (outer dimensions).
template <class F>
RowsArgs<F::N + 1> rows_args(const MapCall &c, int variant) {
    constexpr int NOPS = F::N + 1;
    RowsArgs<NOPS> a{};
    a.n = c.n;
    a.const_mask = 0;
    a.bcast_mask = 0;
    const int last = c.ndim - 1;
    for (int k = 0; k < NOPS; ++k) {
        a.ptr[k] = c.is_const[k] ? c.ptr[0] : c.ptr[k];  // a constant's (ignored) chunk is read from the output
        a.cbits[k] = c.cbits[k];
        if (c.is_const[k]) a.const_mask |= 1u << k;
        else if (c.ndim == 0 || c.stride[k][last] == 0) a.bcast_mask |= k == 0 ? 0u : 1u << k;
    }
    // Eight consecutive tiles are sixteen consecutive output bytes when the output is one run (variant 0) or
    // its rows hold a multiple of eight tiles; the output's base is 16-byte aligned then (pick_variant checks
    // 2-byte alignment only).
    using T = MapTraits<F>;
    a.gather = 0;
    if (T::V * T::so == 2 && reinterpret_cast<uintptr_t>(c.ptr[0]) % 16 == 0) {
        bool whole = variant == 0 || c.size[last] % (8 * T::V) == 0;
        for (int d = 0; whole && variant != 0 && d < last; ++d) whole = (c.stride[0][d] * T::so) % 16 == 0;
        a.gather = whole ? 1u : 0u;
    }
    int64_t span = 1;  // elements from the output's first to one past its last
    for (int d = 0; d < c.ndim; ++d) span += (c.size[d] - 1) * (c.stride[0][d] < 0 ? -c.stride[0][d] : c.stride[0][d]);
    a.out32 = span * T::so <= kNarrowSpanBytes && !(c.n * T::so >= kStreamStoreBytes) ? 1u : 0u;
    if (variant == 0) {
        a.inner = static_cast<uint32_t>(c.n < (int64_t{1} << 31) ? c.n : 0);
        a.nouter = 0;
    } else {
        a.inner = static_cast<uint32_t>(c.size[last]);
        a.inner_div = make_fastdiv(a.inner);
        // The outer dimensions in walking order, innermost first. Any order computes the same elements; the
        // order decides which rows a workgroup touches together.
        struct Outer {
            int64_t size;
            int64_t stride[NOPS];
        } outer[kFastDims];
        int n = 0;
        for (int src = last - 1; src >= 0; --src, ++n) {
            outer[n].size = c.size[src];
            for (int k = 0; k < NOPS; ++k) outer[n].stride[k] = c.is_const[k] ? 0 : c.stride[k][src];
        }
        // A transposed pair (a permuted view copied or mapped into a contiguous tensor): the output runs along
        // dimension 0, an input along dimension 1. Walking a few steps of dimension 0, then dimension 1, then the
        // rest of dimension 0 gives a workgroup's rows runs of that many rows in the output and a few rows in
        // that input, instead of 64 rows in one and single rows in the other. The run is 4 KB of output: measured
        // on [8, 32, S, D] views of 134 MB with rows of 128 bytes to 2 KB, runs of 4 KB are the fastest or within
        // 1 % of it for every row width, and take the same time wherever the buffers lie (runs of 2 KB are as fast
        // for some placements of the output and 3 to 13 % slower for others; 8 KB and more are slower everywhere).
        bool transposed = false;
        if (n >= 2 && n < kFastDims - 1 && outer[1].size >= 8) {
            for (int k = 1; k < NOPS && !transposed; ++k) {
                transposed = !c.is_const[k] && outer[1].stride[k] != 0 && outer[1].stride[k] < outer[0].stride[k] &&
                             outer[0].stride[0] < outer[1].stride[0];
            }
        }
        if (transposed) {
            const int64_t row_bytes = c.size[last] * static_cast<int64_t>(sizeof(typename F::Out));
            int64_t run = 4096 / row_bytes;
            run = run < 4 ? 4 : run > 64 ? 64 : run;
            while (run >= 4 && (outer[0].size % run != 0 || outer[0].size <= run)) run /= 2;
            if (run >= 4) {
                for (int d = n; d > 2; --d) outer[d] = outer[d - 1];
                outer[2] = outer[0];
                outer[2].size = outer[0].size / run;
                for (int k = 0; k < NOPS; ++k) outer[2].stride[k] = outer[0].stride[k] * run;
                outer[0].size = run;
                ++n;
            }
        }
        a.nouter = n;
        for (int d = 0; d < n; ++d) {
            a.div[d] = make_fastdiv(static_cast<uint32_t>(outer[d].size));
            for (int k = 0; k < NOPS; ++k) a.ostride[k][d] = static_cast<int32_t>(outer[d].stride[k]);
        }
    }
    return a;
}

// Whether a call of the general layout is a transposition the tiled kernel takes: the output contiguous along
// its innermost dimension `a`, at least one input contiguous along another dimension `b` (the same for all such
// inputs), every other input contiguous or uniform along `a`; both dimensions long enough to fill tiles. On
// success `b` is that dimension.
template <class F>
bool tiled_applies(const MapCall &c, int &b) {
    using TT = TiledTraits<F>;
    if constexpr (F::N > 2 || TT::lds_bytes > 96 * 1024) {
        return false;
    } else {
        if (c.ndim < 2 || c.ndim > kFastDims || !fits_32(c)) return false;
        const int a = c.ndim - 1;
        if (c.stride[0][a] != 1) return false;
        b = -1;
        for (int k = 1; k < c.nops; ++k) {
            if (c.is_const[k]) continue;
            for (int d = 0; d < c.ndim; ++d) {
                if (c.stride[k][d] < 0) return false;
            }
            if (c.stride[k][a] == 1 || c.stride[k][a] == 0) continue;  // runs with the output
            int along = -1;
            for (int d = 0; d < a; ++d) {
                if (c.stride[k][d] == 1) along = d;
            }
            if (along < 0 || (b >= 0 && along != b)) return false;
            b = along;
        }
        if (b < 0) return false;
        return c.size[a] >= TT::S / 2 && c.size[b] >= TT::S / 2;
    }
}

// Whether a call that tiled_applies accepted (with `b`) can take the 16-byte form: one input turned, the others
// running with the output, both dimensions whole 16-byte slots, every access aligned.
template <class F>
bool tiled16_applies(const MapCall &c, int b) {
    using TT = Tiled16Traits<F>;
    if constexpr (!TT::applies) {
        return false;
    } else {
        const int a = c.ndim - 1;
        // Whole 16-byte slots along both dimensions (the last tiles may be partly empty), and enough of them.
        if (c.size[a] % TT::V != 0 || c.size[b] % TT::V != 0) return false;
        if (c.size[a] < TT::TA / 2 || c.size[b] < TT::TB / 2) return false;
        int turned = 0;
        for (int k = 0; k < c.nops; ++k) {
            if (c.is_const[k]) continue;
            const bool is_turned = k > 0 && c.stride[k][a] != 1;
            if (is_turned) {
                if (c.stride[k][a] == 0 || c.stride[k][b] != 1) return false;
                ++turned;
            }
            if (reinterpret_cast<uintptr_t>(c.ptr[k]) % 16 != 0) return false;
            for (int d = 0; d < c.ndim; ++d) {
                if (d == (is_turned ? b : a)) continue;
                if ((c.stride[k][d] * TT::E) % 16 != 0) return false;
            }
        }
        return turned == 1;
    }
}

template <class F>
void launch_tiled(const MapCall &c, int b, hipStream_t stream) {
    using TT = TiledTraits<F>;
    constexpr int NOPS = F::N + 1;
    if constexpr (F::N <= 2 && TT::lds_bytes <= 96 * 1024) {
        TiledArgs<NOPS> t{};
        const int a = c.ndim - 1;
        const bool wide = tiled16_applies<F>(c, b);
        const uint32_t edge_a = wide ? static_cast<uint32_t>(Tiled16Traits<F>::TA) : static_cast<uint32_t>(TT::S);
        const uint32_t edge_b = wide ? static_cast<uint32_t>(Tiled16Traits<F>::TB) : static_cast<uint32_t>(TT::S);
        t.const_mask = 0;
        t.turned_mask = 0;
        for (int k = 0; k < NOPS; ++k) {
            t.ptr[k] = c.is_const[k] ? c.ptr[0] : c.ptr[k];
            t.cbits[k] = c.cbits[k];
            if (c.is_const[k]) t.const_mask |= 1u << k;
            t.stride_a[k] = c.is_const[k] ? 0 : static_cast<int32_t>(c.stride[k][a]);
            t.stride_b[k] = c.is_const[k] ? 0 : static_cast<int32_t>(c.stride[k][b]);
            if (k > 0 && !c.is_const[k] && c.stride[k][a] != 1 && c.stride[k][a] != 0) t.turned_mask |= 1u << k;
        }
        t.size_a = static_cast<uint32_t>(c.size[a]);
        t.size_b = static_cast<uint32_t>(c.size[b]);
        const uint32_t tiles_a = (t.size_a + edge_a - 1) / edge_a, tiles_b = (t.size_b + edge_b - 1) / edge_b;
        t.tiles_a = make_fastdiv(tiles_a);
        t.tiles_b = make_fastdiv(tiles_b);
        int64_t blocks = static_cast<int64_t>(tiles_a) * tiles_b;
        t.nouter = 0;
        for (int d = c.ndim - 2; d >= 0; --d) {
            if (d == b) continue;
            t.div[t.nouter] = make_fastdiv(static_cast<uint32_t>(c.size[d]));
            for (int k = 0; k < NOPS; ++k) t.ostride[k][t.nouter] = c.is_const[k] ? 0 : static_cast<int32_t>(c.stride[k][d]);
            blocks *= c.size[d];
            ++t.nouter;
        }
        if constexpr (Tiled16Traits<F>::applies) {
            if (wide) {
                // Streaming accesses for calls that do not fit the memory-side cache, as for the rows kernel.
                constexpr int threads = Tiled16Traits<F>::kThreads;
                const int64_t moved = c.n * Tiled16Traits<F>::E * NOPS;
                if (moved > kCacheResidentBytes) {
                    hipLaunchKernelGGL((map_tiled16_kernel<F, true>), dim3(static_cast<unsigned>(blocks)), dim3(threads), 0, stream, t);
                } else {
                    hipLaunchKernelGGL((map_tiled16_kernel<F, false>), dim3(static_cast<unsigned>(blocks)), dim3(threads), 0, stream, t);
                }
                return;
            }
        }
        hipLaunchKernelGGL((map_tiled_kernel<F>), dim3(static_cast<unsigned>(blocks)), dim3(kBlock), 0, stream, t);
    }
}

template <class F>
void launch_map(const MapCall &c, hipStream_t stream) {
    using T = MapTraits<F>;
    constexpr int NOPS = F::N + 1;
    const int variant = resolve_variant<F>(c);
    if (variant <= 1) {
        RowsArgs<NOPS> a = rows_args<F>(c, variant);
        int64_t tiles = (c.n + T::V - 1) / T::V;
        unsigned grid = grid_for(tiles, int64_t{T::U} * kRowsBlock);
        // Which inputs are broadcast (a zero stride in some dimension). Three patterns get kernels of their own:
        // every input (an outer product), the first one only, the second one only (x + bias, x * scale).
        int reused = 0, inputs = 0;
        for (int k = 1; k < NOPS; ++k) {
            if (c.is_const[k]) continue;
            inputs |= 1 << (k - 1);
            for (int d = 0; d < c.ndim; ++d) {
                if (c.stride[k][d] == 0) reused |= 1 << (k - 1);
            }
        }
        auto run = [&](auto flat) {
            constexpr bool kFlat = decltype(flat)::value;
            if constexpr (F::N >= 2) {
                if (inputs != 0 && reused == inputs) {
                    hipLaunchKernelGGL((map_rows_kernel<F, kFlat, 7>), dim3(grid), dim3(kRowsBlock), 0, stream, a);
                    return;
                }
                if (reused == 1) {
                    hipLaunchKernelGGL((map_rows_kernel<F, kFlat, 1>), dim3(grid), dim3(kRowsBlock), 0, stream, a);
                    return;
                }
                if (reused == 2) {
                    hipLaunchKernelGGL((map_rows_kernel<F, kFlat, 2>), dim3(grid), dim3(kRowsBlock), 0, stream, a);
                    return;
                }
                if constexpr (F::N >= 3) {
                    // Two broadcast inputs in front of a streamed one (addr with its input: v1, v2, input).
                    if (reused == 3) {
                        hipLaunchKernelGGL((map_rows_kernel<F, kFlat, 3>), dim3(grid), dim3(kRowsBlock), 0, stream, a);
                        return;
                    }
                }
            }
            hipLaunchKernelGGL((map_rows_kernel<F, kFlat, 0>), dim3(grid), dim3(kRowsBlock), 0, stream, a);
        };
        if (variant == 0) run(std::true_type{});
        else run(std::false_type{});
        return;
    }
    if (variant == 2) {
        int b = -1;
        if (tiled_applies<F>(c, b)) {
            launch_tiled<F>(c, b, stream);
            return;
        }
        // An output that runs along another dimension than the last one (a write into a transposed or permuted
        // view): elements are independent, so the dimensions may be taken in any order; with that dimension
        // last the call is a transposition like any other.
        for (int d = 0; d + 1 < c.ndim; ++d) {
            if (c.stride[0][d] != 1) continue;
            MapCall t = c;
            std::swap(t.size[d], t.size[c.ndim - 1]);
            for (int k = 0; k < c.nops; ++k) std::swap(t.stride[k][d], t.stride[k][c.ndim - 1]);
            if (tiled_applies<F>(t, b)) {
                launch_tiled<F>(t, b, stream);
                return;
            }
            break;
        }
    }
    unsigned grid = grid_for(c.n, variant == 2 ? kAnyPerLane<uint32_t> * kBlock : kBlock);
    if (variant == 2) {
        AnyArgs<NOPS, uint32_t> a{};
        a.n = c.n;
        a.ndim = c.ndim;
        a.const_mask = 0;
        for (int k = 0; k < NOPS; ++k) {
            a.ptr[k] = c.ptr[k];
            a.cbits[k] = c.cbits[k];
            if (c.is_const[k]) a.const_mask |= 1u << k;
        }
        for (int d = 0; d < c.ndim; ++d) {
            int src = c.ndim - 1 - d;
            a.div[d] = make_fastdiv(static_cast<uint32_t>(c.size[src]));
            for (int k = 0; k < NOPS; ++k) a.stride[k][d] = c.is_const[k] ? 0 : static_cast<int32_t>(c.stride[k][src]);
        }
        hipLaunchKernelGGL((map_any_kernel<F, uint32_t>), dim3(grid), dim3(kBlock), 0, stream, a);
    } else {
        AnyArgs<NOPS, int64_t> a{};
        a.n = c.n;
        a.ndim = c.ndim;
        a.const_mask = 0;
        for (int k = 0; k < NOPS; ++k) {
            a.ptr[k] = c.ptr[k];
            a.cbits[k] = c.cbits[k];
            if (c.is_const[k]) a.const_mask |= 1u << k;
        }
        for (int d = 0; d < c.ndim; ++d) {
            int src = c.ndim - 1 - d;
            a.size64[d] = c.size[src];
            for (int k = 0; k < NOPS; ++k) a.stride[k][d] = c.is_const[k] ? 0 : c.stride[k][src];
        }
        hipLaunchKernelGGL((map_any_kernel<F, int64_t>), dim3(grid), dim3(kBlock), 0, stream, a);
    }
}

}  // namespace hmr
