// Reduction machinery for gfx950 (wave64): accumulator ops, wave/block combining and the kernels.
//
// What is computed follows homura's CPU reductions (ref: src/backend/cpu/reduce.rs:43-225): float
// sums/products/means accumulate in f64, integer ones wrap in i64, max/min keep the first NaN and
// then the first of equal values, all/any are truth folds. The order of float additions differs
// from the CPU's sequential order but depends only on sizes and strides, so results repeat
// bit for bit from run to run (ref: csrc/homura_rocm.h:302-303 makes the same promise).
//
// Kernels (the plan in reduce.hip picks one):
//   reduce_rows_kernel  the reduced range is one contiguous run per output ("dim=-1"): one wave,
//                       or one 256-lane workgroup, per output row; 128-bit loads, four in flight
//                       per lane; lanes combine with wave shuffles, waves through LDS.
//   reduce_cols_kernel  outputs are contiguous in memory and the reduced dimension strides over
//                       them ("dim=0"): a lane owns V adjacent columns (one 128-bit load per row)
//                       and the workgroup spans up to 256 lanes * V contiguous columns, so each
//                       row is read in spans of up to 4 KB; row slices are spread over blockIdx.y.
//                       Narrow outputs use fewer waves across and let the others take interleaved
//                       rows, combined through LDS.
//   var_rows_kernel     variance of contiguous rows that fit in registers: the row is read once
//                       and both CPU passes (mean, squared deviations) run on the registers.
//   reduce_any_kernel   any other layout: G lanes per output walk the reduced index space with
//                       div/mod; scalar loads.
// When the reduced range is cut into slices (few outputs, long ranges), each slice leaves a
// partial accumulator in the workspace and a combine kernel folds them in slice order.
//
// An op has two faces. Inside a lane elements arrive in increasing position, one at a time, and
// are folded into a cheap `Lane` state (lane_add). Lane states become `Acc` values (lane_done)
// that `combine` folds across lanes, waves and slices in a fixed order.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>

#include "common.hpp"
#include "elem.hpp"
#include "map.hpp"

namespace hmr {

constexpr int kWave = 64;

// Up to HMR_MAX_DIMS dimensions with one stride set; walks a linear index into an element offset.
struct Walk {
    int32_t ndim;
    int64_t size[HMR_MAX_DIMS];    // innermost first
    int64_t stride[HMR_MAX_DIMS];  // innermost first
    __device__ __forceinline__ int64_t offset(int64_t i) const {
        if (ndim == 1) return i * stride[0];
        int64_t off = 0;
        for (int d = 0; d < ndim; ++d) {
            int64_t q = i / size[d];
            off += (i - q * size[d]) * stride[d];
            i = q;
        }
        return off;
    }
};

// Makes the compiler treat a chunk as newly produced. Kernels that keep a row in registers unpack its chunks again in each phase; without
// this the unpacked values of one phase are kept alive for the next and the packed row costs more
// registers than an unpacked one.
__device__ __forceinline__ void forget(u32x4 &r) { asm volatile("" : "+v"(r)); }

// ---- moving accumulators between lanes ------------------------------------------------------------

template <class A>
__device__ __forceinline__ A shfl_xor_any(A v, int mask) {
    constexpr int words = (sizeof(A) + 3) / 4;
    uint32_t w[words] = {};
    __builtin_memcpy(w, &v, sizeof(A));
#pragma unroll
    for (int i = 0; i < words; ++i) w[i] = static_cast<uint32_t>(__shfl_xor(static_cast<int>(w[i]), mask, kWave));
    A r;
    __builtin_memcpy(&r, w, sizeof(A));
    return r;
}

// Folds the accumulators of the 64 lanes of a wave; every lane ends with the result. The fold is
// a fixed butterfly, so the association order is the same in every run.
template <class Op, class = void>
struct IsCommutative : std::false_type {};
template <class Op>
struct IsCommutative<Op, std::enable_if_t<Op::kCommutative>> : std::true_type {};

template <class Op>
__device__ __forceinline__ typename Op::Acc wave_fold(const Op &op, typename Op::Acc a) {
#pragma unroll
    for (int mask = 1; mask < kWave; mask <<= 1) {
        typename Op::Acc b = shfl_xor_any(a, mask);
        if constexpr (IsCommutative<Op>::value) {
            a = op.combine(a, b);  // combine(a, b) and combine(b, a) have the same bits: both partners agree
        } else {
            // Lower lane first keeps the operand order identical on both partners.
            a = (threadIdx.x & mask) ? op.combine(b, a) : op.combine(a, b);
        }
    }
    return a;
}

// ---- accumulator ops --------------------------------------------------------------------------------

struct NoCtx {};

// Ops whose lane state is the accumulator itself: lane_add(acc, x) = combine(acc, lift(x)).
template <class Derived, class T, class A>
struct SimpleFold {
    using In = T;
    using Acc = A;
    using Lane = A;
    using Ctx = NoCtx;
    __device__ __forceinline__ Ctx context(int64_t) const { return {}; }
    __device__ __forceinline__ Lane lane_init() const { return static_cast<const Derived *>(this)->init(); }
    __device__ __forceinline__ void lane_add(Lane &l, T x, int64_t, Ctx) const {
        const Derived *d = static_cast<const Derived *>(this);
        l = d->combine(l, d->lift(x));
    }
    __device__ __forceinline__ Acc lane_done(const Lane &l) const { return l; }
};

template <class T, bool PROD>
struct FloatFold : SimpleFold<FloatFold<T, PROD>, T, double> {
    static constexpr bool kCommutative = true;  // IEEE + and * are
    __device__ __forceinline__ double init() const { return PROD ? 1.0 : 0.0; }
    __device__ __forceinline__ double lift(T x) const { return Conv<T>::to_f64(x); }
    __device__ __forceinline__ double combine(double a, double b) const { return PROD ? a * b : a + b; }
};

template <class T, bool PROD>
struct IntFold : SimpleFold<IntFold<T, PROD>, T, int64_t> {
    static constexpr bool kCommutative = true;
    __device__ __forceinline__ int64_t init() const { return PROD ? 1 : 0; }
    __device__ __forceinline__ int64_t lift(T x) const { return Conv<T>::to_i64(x); }
    __device__ __forceinline__ int64_t combine(int64_t a, int64_t b) const {
        uint64_t x = static_cast<uint64_t>(a), y = static_cast<uint64_t>(b);
        return static_cast<int64_t>(PROD ? x * y : x + y);
    }
};

template <class T, bool ALL>
struct TruthFold : SimpleFold<TruthFold<T, ALL>, T, uint32_t> {
    static constexpr bool kCommutative = true;
    __device__ __forceinline__ uint32_t init() const { return ALL ? 1u : 0u; }
    __device__ __forceinline__ uint32_t lift(T x) const { return Conv<T>::to_bool(x) ? 1u : 0u; }
    __device__ __forceinline__ uint32_t combine(uint32_t a, uint32_t b) const { return ALL ? (a & b) : (a | b); }
};

// The best element so far and its position in the reduced range (-1: none yet).
template <class T>
struct Best {
    T v;
    int64_t i;
};

// ref: src/backend/cpu/reduce.rs:75-86. Inside a lane positions only grow, so the CPU's scan rule
// applies as it stands: a NaN already held sticks; otherwise a NaN, or a strictly better value,
// replaces. Across lanes the same outcome is: NaN beats non-NaN, better beats worse, and among
// equals (or among NaNs) the lower position wins - associative and commutative.
template <class T, bool MAX>
struct ExtremeFold {
    static constexpr bool kCommutative = true;  // combine picks the same element whichever side it is on
    using In = T;
    using Acc = Best<T>;
    using Lane = Best<T>;
    using Ctx = NoCtx;
    template <class U>
    static __device__ __forceinline__ auto key(U x) {
        if constexpr (std::is_same_v<U, f16_t>) return f16_widen(x);
        else if constexpr (std::is_same_v<U, bf16_t>) return bf16_up(x);
        else if constexpr (std::is_same_v<U, bool_t>) return static_cast<int>(x.v);
        else return x;
    }
    __device__ __forceinline__ Ctx context(int64_t) const { return {}; }
    __device__ __forceinline__ Acc init() const { return Acc{T{}, -1}; }
    __device__ __forceinline__ Lane lane_init() const { return Lane{T{}, -1}; }
    __device__ __forceinline__ void lane_add(Lane &l, T x, int64_t index, Ctx) const {
        auto a = key(l.v), b = key(x);
        // "Not (b <= a)" is one comparison that is true for a better element and for a NaN alike (a held NaN is
        // excluded by a == a). Straight-line code: measured on a column maximum, a wave-wide skip of elements
        // that cannot win (a ballot and a branch per element) cost 130 cycles per element, and so did the same
        // test spelled as (b > a || b != b), which compiles to a chain of mask operations.
        const bool take = l.i < 0 || (a == a && !(MAX ? b <= a : b >= a));
        l.v = take ? x : l.v;
        l.i = take ? index : l.i;
    }
    __device__ __forceinline__ Acc lane_done(const Lane &l) const { return l; }
    __device__ __forceinline__ Acc combine(Acc a, Acc b) const {
        if (b.i < 0) return a;
        if (a.i < 0) return b;
        auto x = key(a.v), y = key(b.v);
        bool xn = x != x, yn = y != y;
        bool a_wins;
        if (xn || yn) a_wins = (xn && yn) ? (a.i < b.i) : xn;
        else if (x == y) a_wins = a.i < b.i;
        else a_wins = MAX ? (x > y) : (x < y);
        return a_wins ? a : b;
    }
};

// Second pass of the two-pass variance: sum of squared deviations from the output's f64 mean.
template <class T>
struct DeviationFold {
    static constexpr bool kCommutative = true;
    using In = T;
    using Acc = double;
    using Lane = double;
    using Ctx = double;
    const double *means;
    __device__ __forceinline__ Ctx context(int64_t o) const { return means[o]; }
    __device__ __forceinline__ Acc init() const { return 0.0; }
    __device__ __forceinline__ Lane lane_init() const { return 0.0; }
    __device__ __forceinline__ void lane_add(Lane &l, T x, int64_t, Ctx mean) const {
        double d = Conv<T>::to_f64(x) - mean;
        l += d * d;
    }
    __device__ __forceinline__ Acc lane_done(const Lane &l) const { return l; }
    __device__ __forceinline__ Acc combine(Acc a, Acc b) const { return a + b; }
};

// One-pass variance for layouts where a second pass would read the source from memory again
// (column reductions). A lane keeps sums of (x - K) and (x - K)^2 about its first element K, which
// is as stable as the two-pass form unless K lies many standard deviations from the mean; lanes,
// waves and slices then merge (count, mean, M2) triples with Chan's update, all in f64. The
// result differs from the CPU's two-pass f64 value by rounding only (a few f64 ulps, a few times n of
// them when K is an outlier of its column), far below one ulp of an f16, bf16 or f32 output; f64
// columns take the two-pass form.
struct Moments {
    double n, mean, m2;
};

// 1 / x for a count x through the hardware reciprocal refined once (relative error about 2^-52). A true
// f64 division is some thirty instructions; the weights of a merge and the mean of a lane do not need it.
__device__ __forceinline__ double count_reciprocal(double x) {
    const double r = __builtin_amdgcn_rcp(x);
    return __builtin_fma(__builtin_fma(-x, r, 1.0), r, r);
}

template <class T>
struct MomentsFold {
    using In = T;
    using Acc = Moments;
    struct Lane {
        double k, s1, s2, n;
    };
    using Ctx = NoCtx;
    __device__ __forceinline__ Ctx context(int64_t) const { return {}; }
    __device__ __forceinline__ Acc init() const { return Acc{0.0, 0.0, 0.0}; }
    __device__ __forceinline__ Lane lane_init() const { return Lane{0.0, 0.0, 0.0, 0.0}; }
    __device__ __forceinline__ void lane_add(Lane &l, T x, int64_t, Ctx) const {
        double v = Conv<T>::to_f64(x);
        l.k = l.n == 0.0 ? v : l.k;
        double d = v - l.k;
        l.s1 += d;
        l.s2 += d * d;
        l.n += 1.0;
    }
    // A whole vector of the row: the shift is settled once for the vector, not once per element.
    template <int V>
    __device__ __forceinline__ void lane_add_vector(Lane &l, const T (&x)[V]) const {
        l.k = l.n == 0.0 ? Conv<T>::to_f64(x[0]) : l.k;
#pragma unroll
        for (int i = 0; i < V; ++i) {
            const double d = Conv<T>::to_f64(x[i]) - l.k;
            l.s1 += d;
            l.s2 += d * d;
        }
        l.n += static_cast<double>(V);
    }
    __device__ __forceinline__ Acc lane_done(const Lane &l) const {
        if (l.n == 0.0) return Acc{0.0, 0.0, 0.0};
        return Acc{l.n, l.k + l.s1 / l.n, l.s2 - l.s1 * l.s1 / l.n};
    }
    __device__ __forceinline__ Acc combine(Acc a, Acc b) const {
        if (b.n == 0.0) return a;
        if (a.n == 0.0) return b;
        const double n = a.n + b.n;
        const double delta = b.mean - a.mean;
        const double wb = b.n * count_reciprocal(n);
        // An infinite mean on either side makes the merged mean infinite, and the deviation of an infinite
        // element from it is inf - inf: the CPU's sum of squares is NaN there, while delta^2 alone would say inf.
        const double poison = delta - delta;  // 0, or NaN when delta is not finite
        return Acc{n, a.mean + delta * wb, a.m2 + b.m2 + delta * delta * (a.n * wb) + poison};
    }
};

// ---- sinks: what happens to a finished accumulator ------------------------------------------------

template <class T, bool MEAN>
struct RoundSink {
    T *out;
    __device__ __forceinline__ void put(int64_t o, double a, int64_t count) const {
        out[o] = Conv<T>::from_f64(MEAN ? a / static_cast<double>(count) : a);
    }
};

struct I64Sink {
    int64_t *out;
    __device__ __forceinline__ void put(int64_t o, int64_t a, int64_t) const { out[o] = a; }
};

struct TruthSink {
    uint8_t *out;
    __device__ __forceinline__ void put(int64_t o, uint32_t a, int64_t) const { out[o] = a != 0; }
};

template <class T>
struct ExtremeSink {
    T *values;         // may be null
    int64_t *indices;  // may be null
    __device__ __forceinline__ void put(int64_t o, Best<T> a, int64_t) const {
        if (values) values[o] = a.v;
        if (indices) indices[o] = a.i;
    }
};

struct MeanSink {
    double *means;
    __device__ __forceinline__ void put(int64_t o, double a, int64_t count) const {
        means[o] = a / static_cast<double>(count);
    }
};

// ref: src/backend/cpu/reduce.rs:160-166: NaN for an empty reduction, else sq / max(0, n - correction).
template <class T>
struct VarSink {
    T *out;
    double divisor;
    bool take_sqrt;
    __device__ __forceinline__ void finish(int64_t o, double sq, int64_t count) const {
        double v = count == 0 ? __builtin_nan("") : sq / divisor;
        out[o] = Conv<T>::from_f64(take_sqrt ? sqrt(v) : v);
    }
    __device__ __forceinline__ void put(int64_t o, double sq, int64_t count) const { finish(o, sq, count); }
    __device__ __forceinline__ void put(int64_t o, Moments m, int64_t count) const { finish(o, m.m2, count); }
};

template <class Acc>
__device__ __forceinline__ void put_partial(void *partials, int64_t nout, int64_t split, int64_t o, Acc a) {
    static_cast<Acc *>(partials)[split * nout + o] = a;
}

// ---- arguments shared by the kernels ----------------------------------------------------------------

// A reduced range made of several contiguous runs (a Rows plan over more than one reduced dimension, one of them
// with stride 1: the statistics of a batch normalisation over [N, C, L], the sum of a transposed view). The runs
// are counted over the other reduced dimensions, innermost first; an element's position in the CPU's order of the
// reduced range (what max/min report) is the sum of its coordinates times `pos`.
constexpr int kRunDims = 3;
struct Runs {
    int32_t dims;               // the other reduced dimensions; 0: the range is one run
    uint32_t length;            // elements of a run, a multiple of the 16-byte vector
    FastDiv vectors;            // 16-byte vectors of a run
    int64_t inner_pos;          // position stride of a run's elements
    FastDiv size[kRunDims];     // the other dimensions ...
    int64_t stride[kRunDims];   // ... their strides in elements ...
    int64_t pos[kRunDims];      // ... and position strides
};

struct ReduceArgs {
    const char *src;  // address of the source's element (offset)
    Walk kept;        // kept dims, source strides
    Walk red;         // reduced dims, source strides
    int64_t nout;
    int64_t nred;
    int64_t splits;   // slices of the reduced range
    int64_t chunk;    // reduced elements per slice
    void *partials;   // workspace for splits > 1
    Runs runs;        // Rows plans only
};

// Sources are read once: every vector load carries the nontemporal hint (a compile-time property of the load;
// a run-time choice between the two forms is merged by the compiler into one plain load).
template <class T, int V>
__device__ __forceinline__ void load_stream(const char *p, T (&r)[V]) {
    load_tile<T, V, kStreamLoads>(p, r);
}

// ---- kernels -----------------------------------------------------------------------------------------

// G lanes per output (G = 1, 64 or 256), any layout.
template <class Op, class Sink, int G>
__global__ void __launch_bounds__(kBlock) reduce_any_kernel(ReduceArgs a, Op op, Sink sink) {
    using T = typename Op::In;
    using Acc = typename Op::Acc;
    constexpr int kPerBlock = kBlock / G;
    __shared__ Acc lds[G == kBlock ? kBlock / kWave : 1];
    const int lane = threadIdx.x % G;
    const int64_t split = blockIdx.y;
    const int64_t begin = split * a.chunk;
    const int64_t end = begin + a.chunk < a.nred ? begin + a.chunk : a.nred;
    const int64_t groups = (a.nout + kPerBlock - 1) / kPerBlock;
    for (int64_t g = blockIdx.x; g < groups; g += gridDim.x) {
        const int64_t o = g * kPerBlock + threadIdx.x / G;
        const bool live = o < a.nout;
        typename Op::Lane state = op.lane_init();
        if (live) {
            const typename Op::Ctx ctx = op.context(o);
            const T *p = reinterpret_cast<const T *>(a.src) + a.kept.offset(o);
            for (int64_t r = begin + lane; r < end; r += G) op.lane_add(state, p[a.red.offset(r)], r, ctx);
        }
        Acc acc = op.lane_done(state);
        if constexpr (G >= kWave) acc = wave_fold(op, acc);
        if constexpr (G == kBlock) {
            __syncthreads();  // lds reuse across iterations
            if (threadIdx.x % kWave == 0) lds[threadIdx.x / kWave] = acc;
            __syncthreads();
            acc = lds[0];
#pragma unroll
            for (int w = 1; w < kBlock / kWave; ++w) acc = op.combine(acc, lds[w]);
        }
        if (live && lane == 0) {
            if (a.splits > 1) put_partial(a.partials, a.nout, split, o, acc);
            else sink.put(o, acc, a.nred);
        }
    }
}

// Folds the slices of each output, in an order fixed by the sizes alone. A workgroup takes OUTS
// adjacent outputs (64, 16, 4 or 1: the fewer outputs there are, the fewer each workgroup takes, so
// that the grid still covers the GPU); its 256 lanes are 256/OUTS slice lanes per output. A lane folds
// every (256/OUTS)-th slice, four loads in flight; the slice lanes of an output that share a wave meet
// by shuffles, the four waves through LDS.
template <class Op, class Sink, int OUTS>
__global__ void __launch_bounds__(kBlock) combine_kernel(ReduceArgs a, Op op, Sink sink) {
    using Acc = typename Op::Acc;
    constexpr int kWaves = kBlock / kWave;
    constexpr int L = kBlock / OUTS;  // slice lanes per output
    constexpr int U = 4;
    __shared__ Acc lds[kWaves - 1][kWave];
    const Acc *partials = static_cast<const Acc *>(a.partials);
    const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
    const int ol = threadIdx.x % OUTS, sl = threadIdx.x / OUTS;
    const int64_t groups = (a.nout + OUTS - 1) / OUTS;
    for (int64_t g = blockIdx.x; g < groups; g += gridDim.x) {
        const int64_t o = g * OUTS + ol;
        Acc acc = op.init();
        if (o < a.nout) {
            // Batches of U loads, all issued before the first is folded (a slice past the end reads the last
            // slice again and is left out): a lane's slices cost one trip to memory per batch, not one each.
            for (int64_t s = sl; s < a.splits; s += U * L) {
                Acc t[U];
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    const int64_t k = s + u * L < a.splits ? s + u * L : a.splits - 1;
                    t[u] = partials[k * a.nout + o];
                }
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    if (s + u * L < a.splits) acc = op.combine(acc, t[u]);
                }
            }
        }
        // Slice lanes of one output inside a wave sit OUTS lanes apart.
#pragma unroll
        for (int mask = OUTS; mask < kWave; mask <<= 1) {
            Acc other = shfl_xor_any(acc, mask);
            if constexpr (IsCommutative<Op>::value) acc = op.combine(acc, other);
            else acc = (lane & mask) ? op.combine(other, acc) : op.combine(acc, other);
        }
        __syncthreads();
        if (wave > 0) lds[wave - 1][lane] = acc;
        __syncthreads();
        if (wave == 0 && lane < OUTS && o < a.nout) {
#pragma unroll
            for (int w = 0; w < kWaves - 1; ++w) acc = op.combine(acc, lds[w][lane]);
            sink.put(o, acc, a.nred);
        }
    }
}

// Contiguous rows, each starting 16-byte aligned. WAVES = 1: a wave per row, four rows per
// workgroup. WAVES = 4: a workgroup per row (or per row slice when splits > 1).
// The V elements of one vector into a lane's state: through the op's own vector form when it has one (the
// elements' positions do not matter to such an op), else one by one with positions `pos + i * step`.
template <class Op, class = void>
struct HasVectorAdd : std::false_type {};
template <class Op>
struct HasVectorAdd<Op, std::void_t<decltype(&Op::template lane_add_vector<2>)>> : std::true_type {};

template <class Op, int V>
__device__ __forceinline__ void add_vector(const Op &op, typename Op::Lane &state, const typename Op::In (&x)[V], int64_t pos,
                                           int64_t step, typename Op::Ctx ctx) {
    if constexpr (HasVectorAdd<Op>::value) {
        op.template lane_add_vector<V>(state, x);
    } else {
#pragma unroll
        for (int i = 0; i < V; ++i) op.lane_add(state, x[i], pos + i * step, ctx);
    }
}

template <class Op, class Sink, int WAVES>
__global__ void __launch_bounds__(kBlock) reduce_rows_kernel(ReduceArgs a, Op op, Sink sink) {
    using T = typename Op::In;
    using Acc = typename Op::Acc;
    constexpr int V = 16 / static_cast<int>(sizeof(T));
    constexpr int G = WAVES * kWave;
    constexpr int kPerBlock = kBlock / G;
    constexpr int U = 4;  // loads in flight per lane
    __shared__ Acc lds[WAVES == 4 ? 4 : 1];
    const int lane = threadIdx.x % G;
    const int64_t split = blockIdx.y;
    const int64_t begin = split * a.chunk;
    const int64_t end = begin + a.chunk < a.nred ? begin + a.chunk : a.nred;
    const int64_t groups = (a.nout + kPerBlock - 1) / kPerBlock;
    for (int64_t g = blockIdx.x; g < groups; g += gridDim.x) {
        const int64_t o = g * kPerBlock + threadIdx.x / G;
        const bool live = o < a.nout;
        typename Op::Lane state = op.lane_init();
        if (live) {
            const typename Op::Ctx ctx = op.context(o);
            const T *p = reinterpret_cast<const T *>(a.src) + a.kept.offset(o);
            // Whole vectors: positions begin + (lane + k*G)*V.
            const int64_t nvec = (end - begin) / V;
            int64_t k = lane;
            if (a.runs.dims > 0) {
                // Several runs: vector number -> (run, vector inside it) by a 32-bit division, the run's start
                // and its first position from its coordinates. Slices are whole vectors, runs too.
                const uint32_t v0 = static_cast<uint32_t>(begin / V);
                auto locate = [&](uint32_t v, int64_t &at, int64_t &pos) {
                    uint32_t run = divide(v, a.runs.vectors);
                    const uint32_t inside = (v - run * a.runs.vectors.div) * V;
                    at = inside;
                    pos = inside * a.runs.inner_pos;
                    for (int d = 0; d < a.runs.dims; ++d) {
                        const uint32_t q = divide(run, a.runs.size[d]);
                        const int64_t c = run - q * a.runs.size[d].div;
                        run = q;
                        at += c * a.runs.stride[d];
                        pos += c * a.runs.pos[d];
                    }
                };
                for (; k + (U - 1) * G < nvec; k += U * G) {
                    T r[U][V];
                    int64_t pos[U];
#pragma unroll
                    for (int u = 0; u < U; ++u) {
                        int64_t at;
                        locate(v0 + static_cast<uint32_t>(k + u * G), at, pos[u]);
                        load_stream<T, V>(reinterpret_cast<const char *>(p + at), r[u]);
                    }
#pragma unroll
                    for (int u = 0; u < U; ++u) {
                        add_vector<Op, V>(op, state, r[u], pos[u], a.runs.inner_pos, ctx);
                    }
                }
                for (; k < nvec; k += G) {
                    T r[V];
                    int64_t at, pos;
                    locate(v0 + static_cast<uint32_t>(k), at, pos);
                    load_stream<T, V>(reinterpret_cast<const char *>(p + at), r);
                    add_vector<Op, V>(op, state, r, pos, a.runs.inner_pos, ctx);
                }
                k = nvec;  // nothing ragged: the range is whole runs
            }
            for (; k + (U - 1) * G < nvec; k += U * G) {
                T r[U][V];
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    load_stream<T, V>(reinterpret_cast<const char *>(p + begin + (k + u * G) * V), r[u]);
                }
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    add_vector<Op, V>(op, state, r[u], begin + (k + u * G) * V, 1, ctx);
                }
            }
            for (; k < nvec; k += G) {
                T r[V];
                load_stream<T, V>(reinterpret_cast<const char *>(p + begin + k * V), r);
                add_vector<Op, V>(op, state, r, begin + k * V, 1, ctx);
            }
            // Ragged end of the range (fewer than V elements; one run only).
            if (a.runs.dims == 0) {
                for (int64_t r = begin + nvec * V + lane; r < end; r += G) op.lane_add(state, p[r], r, ctx);
            }
        }
        Acc acc = wave_fold(op, op.lane_done(state));
        if constexpr (WAVES == 4) {
            __syncthreads();
            if (threadIdx.x % kWave == 0) lds[threadIdx.x / kWave] = acc;
            __syncthreads();
            acc = lds[0];
#pragma unroll
            for (int w = 1; w < 4; ++w) acc = op.combine(acc, lds[w]);
        }
        if (live && lane == 0) {
            if (a.splits > 1) put_partial(a.partials, a.nout, split, o, acc);
            else sink.put(o, acc, a.nred);
        }
    }
}

// ---- the column kernel ----------------------------------------------------------------------------
//
// Per-column state of a lane of the column kernel. The kernel feeds a lane the rows of its columns in
// increasing order, the first one through `first`, which seeds the state, so that the update of the
// following rows tests nothing about emptiness; row numbers are 32-bit (the plan keeps the column kernel
// below 2^31 rows) and the kernel knows how many rows it fed when it asks for the accumulator.
template <class Op, class = void>
struct ColState {
    using T = typename Op::In;
    typename Op::Lane s;
    __device__ __forceinline__ void first(const Op &op, T x, int32_t r, typename Op::Ctx c) {
        s = op.lane_init();
        op.lane_add(s, x, r, c);
    }
    __device__ __forceinline__ void next(const Op &op, T x, int32_t r, typename Op::Ctx c) { op.lane_add(s, x, r, c); }
    __device__ __forceinline__ typename Op::Acc done(const Op &op, int32_t) const { return op.lane_done(s); }
};

template <class T, bool MAX>
struct ColState<ExtremeFold<T, MAX>> {
    using Op = ExtremeFold<T, MAX>;
    T v;
    int32_t i;
    __device__ __forceinline__ void first(const Op &, T x, int32_t r, NoCtx) {
        v = x;
        i = r;
    }
    // ref: src/backend/cpu/reduce.rs:75-86 with positions that only grow: a held NaN sticks (a == a fails),
    // otherwise a NaN or a strictly better value replaces ("not (b <= a)" is true for both).
    __device__ __forceinline__ void next(const Op &, T x, int32_t r, NoCtx) {
        auto a = Op::key(v), b = Op::key(x);
        const bool take = a == a && !(MAX ? b <= a : b >= a);
        v = take ? x : v;
        i = take ? r : i;
    }
    __device__ __forceinline__ Best<T> done(const Op &, int32_t) const { return Best<T>{v, static_cast<int64_t>(i)}; }
};

// Sums of (x - K) and (x - K)^2 about the lane's first element K (see MomentsFold): the count is the
// kernel's, the squares go through one fused multiply-add (nothing here has to match the CPU's roundings;
// the result is judged against its two-pass value).
template <class T>
struct ColState<MomentsFold<T>> {
    using Op = MomentsFold<T>;
    double k, s1, s2;
    __device__ __forceinline__ void first(const Op &, T x, int32_t, NoCtx) {
        k = Conv<T>::to_f64(x);
        s1 = 0.0;
        s2 = k - k;  // 0, or NaN when the element is an infinity or a NaN: its deviation from itself, as the CPU has it
    }
    __device__ __forceinline__ void next(const Op &, T x, int32_t, NoCtx) {
        const double d = Conv<T>::to_f64(x) - k;
        s1 += d;
        s2 = __builtin_fma(d, d, s2);
    }
    __device__ __forceinline__ Moments done(const Op &, int32_t count) const {
        const double n = static_cast<double>(count);
        const double mean_shift = s1 * count_reciprocal(n);
        const double m2 = s2 - s1 * mean_shift;
        return Moments{n, k + mean_shift, m2 < 0.0 ? 0.0 : m2};  // a NaN stays one
    }
};

// Contiguous outputs ("columns"), one strided reduced dimension of fewer than 2^31 rows. `rstride` is that
// stride and `inner` the length of the contiguous run of outputs (the innermost kept dimension); a.kept holds
// the remaining, outer kept dimensions. Every row of every tile starts 16-byte aligned.
//
// A lane owns V adjacent columns (one 16-byte load per row) and keeps their states in registers; `across`
// (1, 2 or 4) waves of the workgroup sit side by side on a span of across*64*V columns and the BLOCK/64/across
// row groups take interleaved rows. The S = gridDim.y slices are interleaved as well: row group g of slice s
// takes rows s*RG + g, s*RG + g + S*RG, ... - so all workgroups of a launch together sweep ONE band of
// S*RG consecutive rows through the source, the way a copy would. (Measured on 16384 x 4096 f32: slices that
// are blocks of consecutive rows, i.e. S streams 4 MB apart, 45.4 us; interleaved 43.1 us.)
// The loop is software-pipelined two rows deep: the next two loads are issued before the last two are folded
// (two rows per step 40.5 us, four 41.8, one 44.1 in that shape).
template <class Op, class Sink, int BLOCK>
__global__ void __launch_bounds__(BLOCK)
    reduce_cols_kernel(ReduceArgs a, int64_t rstride, int64_t inner, int across, Op op, Sink sink) {
    using T = typename Op::In;
    using Acc = typename Op::Acc;
    constexpr int V = 16 / static_cast<int>(sizeof(T));
    constexpr int kWaves = BLOCK / kWave;
    constexpr int U = 2;
    __shared__ Acc lds[kWaves][kWave * V];  // a wave's accumulators, for the fold across row groups
    // The wave's number is the same in all its lanes; said so, the row bookkeeping below (first row, count,
    // the loop itself) stays in scalar registers.
    const int wave = __builtin_amdgcn_readfirstlane(static_cast<int>(threadIdx.x) / kWave), lane = threadIdx.x % kWave;
    const int cgroup = wave % across, rgroup = wave / across, rgroups = kWaves / across;
    // Rows of this wave: first, first + stride, ...
    const int32_t nred = static_cast<int32_t>(a.nred);
    const int32_t stride = static_cast<int32_t>(gridDim.y) * rgroups;
    const int32_t first = static_cast<int32_t>(blockIdx.y) * rgroups + rgroup;
    const int32_t count = first < nred ? (nred - first + stride - 1) / stride : 0;
    const int64_t step = static_cast<int64_t>(stride) * rstride * static_cast<int64_t>(sizeof(T));  // bytes
    const int64_t span = static_cast<int64_t>(across) * kWave * V;
    const int64_t tiles_inner = (inner + span - 1) / span;
    const int64_t tiles = tiles_inner * (a.nout / inner);
    for (int64_t tile = blockIdx.x; tile < tiles; tile += gridDim.x) {
        const int64_t outer = tile / tiles_inner;
        const int64_t col = (tile - outer * tiles_inner) * span + (cgroup * kWave + lane) * V;  // within the run
        const int64_t obase = outer * inner;                                                    // first output of the run
        const T *src = reinterpret_cast<const T *>(a.src) + a.kept.offset(outer);
        const int valid = inner - col >= V ? V : (inner > col ? static_cast<int>(inner - col) : 0);
        ColState<Op> state[V];
        typename Op::Ctx ctx[V];
#pragma unroll
        for (int i = 0; i < V; ++i) ctx[i] = op.context(i < valid ? obase + col + i : 0);
        Acc acc[V];
        if (count > 0 && valid == V) {
            const char *p = reinterpret_cast<const char *>(src + static_cast<int64_t>(first) * rstride + col);
            int32_t r = first, n = count - 1;
            {
                T t[V];
                load_stream<T, V>(p, t);
                p += step;
#pragma unroll
                for (int i = 0; i < V; ++i) state[i].first(op, t[i], r, ctx[i]);
                r += stride;
            }
            auto fold = [&](const T(&t)[V]) {
#pragma unroll
                for (int i = 0; i < V; ++i) state[i].next(op, t[i], r, ctx[i]);
                r += stride;
            };
            // The next U rows are requested before the last U are folded, and handed over by a register copy
            // that waits for them: at most U loads are out per wave at any time. (Two buffers that swap roles keep
            // up to 2 U loads out and measured 1 us slower on 16384 x 4096: this access pattern runs best with
            // little in flight.)
            if (n >= U) {
                T cur[U][V];
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    load_stream<T, V>(p, cur[u]);
                    p += step;
                }
                for (n -= U; n >= U; n -= U) {
                    T nxt[U][V];
#pragma unroll
                    for (int u = 0; u < U; ++u) {
                        load_stream<T, V>(p, nxt[u]);
                        p += step;
                    }
#pragma unroll
                    for (int u = 0; u < U; ++u) fold(cur[u]);
#pragma unroll
                    for (int u = 0; u < U; ++u) {
#pragma unroll
                        for (int i = 0; i < V; ++i) cur[u][i] = nxt[u][i];
                    }
                }
#pragma unroll
                for (int u = 0; u < U; ++u) fold(cur[u]);
            }
            for (; n > 0; --n) {
                T t[V];
                load_stream<T, V>(p, t);
                p += step;
                fold(t);
            }
#pragma unroll
            for (int i = 0; i < V; ++i) acc[i] = state[i].done(op, count);
        } else if (count > 0 && valid > 0) {
            // The ragged last lane of a run of outputs: element by element.
            const T *q = src + static_cast<int64_t>(first) * rstride + col;
            const int64_t estep = static_cast<int64_t>(stride) * rstride;
#pragma unroll
            for (int i = 0; i < V; ++i) {
                if (i < valid) state[i].first(op, q[i], first, ctx[i]);
            }
            int32_t r = first + stride;
            for (int32_t n = count - 1; n > 0; --n, r += stride) {
                q += estep;
#pragma unroll
                for (int i = 0; i < V; ++i) {
                    if (i < valid) state[i].next(op, q[i], r, ctx[i]);
                }
            }
#pragma unroll
            for (int i = 0; i < V; ++i) acc[i] = i < valid ? state[i].done(op, count) : op.init();
        } else {
#pragma unroll
            for (int i = 0; i < V; ++i) acc[i] = op.init();
        }
        const int64_t tile_col = (tile - outer * tiles_inner) * span;  // first column of the tile, within the run
        if (rgroups > 1) {
            // Every wave leaves its accumulators in LDS; then the row groups share the fold: of the 64*V columns
            // of its column group, row group g folds columns [g, g + 1) * 64*V / rgroups, a column per lane, the
            // row groups' values in order. All waves work, and a wave's results are consecutive outputs.
            __syncthreads();  // the previous tile's fold has read LDS
#pragma unroll
            for (int i = 0; i < V; ++i) lds[wave][lane * V + i] = acc[i];
            __syncthreads();
            const int share = kWave * V / rgroups;
            for (int j = lane; j < share; j += kWave) {
                const int c = rgroup * share + j;  // column within the column group
                Acc folded = lds[cgroup][c];
                for (int g = 1; g < rgroups; ++g) folded = op.combine(folded, lds[g * across + cgroup][c]);
                const int64_t column = tile_col + cgroup * (kWave * V) + c;
                if (column < inner) {
                    if (a.splits > 1) put_partial(a.partials, a.nout, static_cast<int64_t>(blockIdx.y), obase + column, folded);
                    else sink.put(obase + column, folded, a.nred);
                }
            }
        } else {
#pragma unroll
            for (int i = 0; i < V; ++i) {
                if (i < valid) {
                    if (a.splits > 1) put_partial(a.partials, a.nout, static_cast<int64_t>(blockIdx.y), obase + col + i, acc[i]);
                    else sink.put(obase + col + i, acc[i], a.nred);
                }
            }
        }
    }
}

// Variance of contiguous, 16-byte aligned rows of G*C*V elements at most, a multiple of V: the row
// is read once into registers (C 16-byte chunks per lane, all loads issued back to back and
// unconditionally - a chunk past the row's end re-reads the last chunk and is left out of the sums),
// then the CPU's two passes run on them (ref: src/backend/cpu/reduce.rs:150-166): mean = sum / n in
// f64, then the sum of squared deviations from that mean.
template <class T, int WAVES, int C>
__global__ void __launch_bounds__(kBlock) var_rows_kernel(ReduceArgs a, VarSink<T> sink) {
    constexpr int V = 16 / static_cast<int>(sizeof(T));
    constexpr int G = WAVES * kWave;
    constexpr int kPerBlock = kBlock / G;
    __shared__ double lds[WAVES == 4 ? 4 : 1];
    const int lane = threadIdx.x % G;
    const FloatFold<T, false> add{};
    const int64_t groups = (a.nout + kPerBlock - 1) / kPerBlock;
    const int nvec = static_cast<int>(a.nred / V);
    auto fold = [&](double v) {
        v = wave_fold(add, v);
        if constexpr (WAVES == 4) {
            __syncthreads();
            if (threadIdx.x % kWave == 0) lds[threadIdx.x / kWave] = v;
            __syncthreads();
            v = lds[0];
#pragma unroll
            for (int w = 1; w < 4; ++w) v += lds[w];
        }
        return v;
    };
    for (int64_t g = blockIdx.x; g < groups; g += gridDim.x) {
        const int64_t o = g * kPerBlock + threadIdx.x / G;
        const bool live = o < a.nout;
        const char *p = a.src + a.kept.offset(live ? o : a.nout - 1) * static_cast<int64_t>(sizeof(T));
        u32x4 raw[C];
#pragma unroll
        for (int c = 0; c < C; ++c) {
            const uint32_t tile = static_cast<uint32_t>(c * G + lane);
            const uint32_t t = tile < static_cast<uint32_t>(nvec) ? tile : static_cast<uint32_t>(nvec - 1);
            const u32x4 *q = reinterpret_cast<const u32x4 *>(p + t * 16u);
            if constexpr (kStreamLoads) raw[c] = __builtin_nontemporal_load(q);
            else raw[c] = *q;
        }
        __builtin_amdgcn_sched_barrier(0);  // every load is out before anything waits for one
        double sum = 0.0;
#pragma unroll
        for (int c = 0; c < C; ++c) {
            T x[V];
            __builtin_memcpy(x, &raw[c], 16);
            double part = 0.0;
#pragma unroll
            for (int i = 0; i < V; ++i) part += Conv<T>::to_f64(x[i]);
            // Lane-local order: chunk by chunk, left to right inside a chunk.
            sum += c * G + lane < nvec ? part : 0.0;
        }
        const double mean = fold(sum) / static_cast<double>(a.nred);
        double sq = 0.0;
#pragma unroll
        for (int c = 0; c < C; ++c) {
            T x[V];
            forget(raw[c]);  // convert again rather than keep every f64 value of the first pass
            __builtin_memcpy(x, &raw[c], 16);
            double part = 0.0;
#pragma unroll
            for (int i = 0; i < V; ++i) {
                const double d = Conv<T>::to_f64(x[i]) - mean;
                part += d * d;
            }
            sq += c * G + lane < nvec ? part : 0.0;
        }
        sq = fold(sq);
        if (live && lane == 0) sink.finish(o, sq, a.nred);
    }
}

}  // namespace hmr
