// Reduction machinery for gfx950 (wave64): accumulator ops, wave/block combining and three kernels.
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
//                       them ("dim=0"): a lane owns V adjacent columns (one 128-bit load per row),
//                       the four waves of a workgroup take interleaved rows of a row slice and
//                       combine through LDS; row slices are spread over blockIdx.y.
//   reduce_any_kernel   any other layout: G lanes per output walk the reduced index space with
//                       div/mod; scalar loads.
// When the reduced range is cut into slices (few outputs, long ranges), each slice leaves a
// partial accumulator in the workspace and combine_kernel folds them in slice order.
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
template <class Op>
__device__ __forceinline__ typename Op::Acc wave_fold(const Op &op, typename Op::Acc a) {
#pragma unroll
    for (int mask = 1; mask < kWave; mask <<= 1) {
        typename Op::Acc b = shfl_xor_any(a, mask);
        // Lower lane first keeps the operand order identical on both partners.
        a = (threadIdx.x & mask) ? op.combine(b, a) : op.combine(a, b);
    }
    return a;
}

// ---- accumulator ops --------------------------------------------------------------------------------
// Acc lift(T x, int64 index, Ctx) turns the element at reduced position `index` into an
// accumulator; combine(a, b) folds two (a's elements come from lower lanes/slices).

struct NoCtx {};

template <class T, bool PROD>
struct FloatFold {
    using In = T;
    using Acc = double;
    using Ctx = NoCtx;
    __device__ __forceinline__ Ctx context(int64_t) const { return {}; }
    __device__ __forceinline__ Acc init() const { return PROD ? 1.0 : 0.0; }
    __device__ __forceinline__ Acc lift(T x, int64_t, Ctx) const { return Conv<T>::to_f64(x); }
    __device__ __forceinline__ Acc combine(Acc a, Acc b) const { return PROD ? a * b : a + b; }
};

template <class T, bool PROD>
struct IntFold {
    using In = T;
    using Acc = int64_t;
    using Ctx = NoCtx;
    __device__ __forceinline__ Ctx context(int64_t) const { return {}; }
    __device__ __forceinline__ Acc init() const { return PROD ? 1 : 0; }
    __device__ __forceinline__ Acc lift(T x, int64_t, Ctx) const { return Conv<T>::to_i64(x); }
    __device__ __forceinline__ Acc combine(Acc a, Acc b) const {
        uint64_t x = static_cast<uint64_t>(a), y = static_cast<uint64_t>(b);
        return static_cast<int64_t>(PROD ? x * y : x + y);
    }
};

template <class T, bool ALL>
struct TruthFold {
    using In = T;
    using Acc = uint32_t;
    using Ctx = NoCtx;
    __device__ __forceinline__ Ctx context(int64_t) const { return {}; }
    __device__ __forceinline__ Acc init() const { return ALL ? 1u : 0u; }
    __device__ __forceinline__ Acc lift(T x, int64_t, Ctx) const { return Conv<T>::to_bool(x) ? 1u : 0u; }
    __device__ __forceinline__ Acc combine(Acc a, Acc b) const { return ALL ? (a & b) : (a | b); }
};

// The best element so far and its position in the reduced range (-1: none yet). The rule of
// ref: src/backend/cpu/reduce.rs:75-86 for a sequential scan - the first NaN wins and sticks,
// otherwise a strictly better value replaces - is the same as: NaN beats non-NaN, better value
// beats worse, and among equals (or among NaNs) the lower position wins. That form is
// associative and commutative, so lanes may combine in any order.
template <class T>
struct Best {
    T v;
    int64_t i;
};

template <class T, bool MAX>
struct ExtremeFold {
    using In = T;
    using Acc = Best<T>;
    using Ctx = NoCtx;
    __device__ __forceinline__ Ctx context(int64_t) const { return {}; }
    __device__ __forceinline__ Acc init() const { return Acc{T{}, -1}; }
    __device__ __forceinline__ Acc lift(T x, int64_t index, Ctx) const { return Acc{x, index}; }
    __device__ __forceinline__ Acc combine(Acc a, Acc b) const {
        if (b.i < 0) return a;
        if (a.i < 0) return b;
        auto x = cmp_key(a.v), y = cmp_key(b.v);
        bool xn = x != x, yn = y != y;
        bool a_wins;
        if (xn || yn) a_wins = (xn && yn) ? (a.i < b.i) : xn;
        else if (x == y) a_wins = a.i < b.i;
        else a_wins = MAX ? (x > y) : (x < y);
        return a_wins ? a : b;
    }
    template <class U>
    static __device__ __forceinline__ auto cmp_key(U x) {
        if constexpr (std::is_same_v<U, f16_t>) return f16_widen(x);
        else if constexpr (std::is_same_v<U, bf16_t>) return bf16_up(x);
        else if constexpr (std::is_same_v<U, bool_t>) return static_cast<int>(x.v);
        else return x;
    }
};

// Second pass of the variance: sum of squared deviations from the output's f64 mean.
template <class T>
struct DeviationFold {
    using In = T;
    using Acc = double;
    using Ctx = double;
    const double *means;
    __device__ __forceinline__ Ctx context(int64_t o) const { return means[o]; }
    __device__ __forceinline__ Acc init() const { return 0.0; }
    __device__ __forceinline__ Acc lift(T x, int64_t, Ctx mean) const {
        double d = Conv<T>::to_f64(x) - mean;
        return d * d;
    }
    __device__ __forceinline__ Acc combine(Acc a, Acc b) const { return a + b; }
};

// ---- sinks: what happens to a finished accumulator ------------------------------------------------

// Rounds a float fold to the dtype (dividing by the count first for a mean).
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

// The f64 mean of each output, kept for the deviation pass.
struct MeanSink {
    double *means;
    __device__ __forceinline__ void put(int64_t o, double a, int64_t count) const {
        means[o] = a / static_cast<double>(count);
    }
};

template <class T>
struct VarSink {
    T *out;
    double divisor;
    bool take_sqrt;
    __device__ __forceinline__ void put(int64_t o, double sq, int64_t count) const {
        double v = count == 0 ? __builtin_nan("") : sq / divisor;
        out[o] = Conv<T>::from_f64(take_sqrt ? sqrt(v) : v);
    }
};

// Writes slice `split` of output o into the workspace instead of finishing it.
template <class Acc>
__device__ __forceinline__ void put_partial(void *partials, int64_t nout, int64_t split, int64_t o, Acc a) {
    static_cast<Acc *>(partials)[split * nout + o] = a;
}

// ---- arguments shared by the kernels ----------------------------------------------------------------

struct ReduceArgs {
    const char *src;  // address of the source's element (offset)
    Walk kept;        // kept dims, source strides
    Walk red;         // reduced dims, source strides
    int64_t nout;
    int64_t nred;
    int64_t splits;   // slices of the reduced range
    int64_t chunk;    // reduced elements per slice
    void *partials;   // workspace for splits > 1
};

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
        Acc acc = op.init();
        if (live) {
            const typename Op::Ctx ctx = op.context(o);
            const T *p = reinterpret_cast<const T *>(a.src) + a.kept.offset(o);
            for (int64_t r = begin + lane; r < end; r += G) acc = op.combine(acc, op.lift(p[a.red.offset(r)], r, ctx));
        }
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

template <class Op, class Sink>
__global__ void __launch_bounds__(kBlock) combine_kernel(ReduceArgs a, Op op, Sink sink) {
    using Acc = typename Op::Acc;
    const Acc *partials = static_cast<const Acc *>(a.partials);
    for (int64_t o = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x; o < a.nout;
         o += static_cast<int64_t>(gridDim.x) * kBlock) {
        Acc acc = partials[o];
        for (int64_t s = 1; s < a.splits; ++s) acc = op.combine(acc, partials[s * a.nout + o]);
        sink.put(o, acc, a.nred);
    }
}

// The same with a wave per output, for few outputs cut into many slices (a full reduction).
template <class Op, class Sink>
__global__ void __launch_bounds__(kBlock) combine_wave_kernel(ReduceArgs a, Op op, Sink sink) {
    using Acc = typename Op::Acc;
    const Acc *partials = static_cast<const Acc *>(a.partials);
    const int lane = threadIdx.x % kWave;
    const int64_t groups = (a.nout + 3) / 4;
    for (int64_t g = blockIdx.x; g < groups; g += gridDim.x) {
        const int64_t o = g * 4 + threadIdx.x / kWave;
        Acc acc = op.init();
        if (o < a.nout) {
            for (int64_t s = lane; s < a.splits; s += kWave) acc = op.combine(acc, partials[s * a.nout + o]);
        }
        acc = wave_fold(op, acc);
        if (o < a.nout && lane == 0) sink.put(o, acc, a.nred);
    }
}

// Contiguous rows. WAVES = 1: a wave per row, four rows per workgroup. WAVES = 4: a workgroup per
// row (or per row slice when splits > 1). VEC: rows start 16-byte aligned, so 128-bit loads.
template <class Op, class Sink, int WAVES, bool VEC>
__global__ void __launch_bounds__(kBlock) reduce_rows_kernel(ReduceArgs a, Op op, Sink sink) {
    using T = typename Op::In;
    using Acc = typename Op::Acc;
    constexpr int V = VEC ? 16 / static_cast<int>(sizeof(T)) : 1;
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
        Acc acc = op.init();
        if (live) {
            const typename Op::Ctx ctx = op.context(o);
            const T *p = reinterpret_cast<const T *>(a.src) + a.kept.offset(o);
            // Whole vectors: positions begin + (lane + k*G)*V.
            const int64_t nvec = (end - begin) / V;
            int64_t k = lane;
            for (; k + (U - 1) * G < nvec; k += U * G) {
                T r[U][V];
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    load_tile<T, V>(reinterpret_cast<const char *>(p + begin + (k + u * G) * V), r[u]);
                }
#pragma unroll
                for (int u = 0; u < U; ++u) {
#pragma unroll
                    for (int i = 0; i < V; ++i) {
                        acc = op.combine(acc, op.lift(r[u][i], begin + (k + u * G) * V + i, ctx));
                    }
                }
            }
            for (; k < nvec; k += G) {
                T r[V];
                load_tile<T, V>(reinterpret_cast<const char *>(p + begin + k * V), r);
#pragma unroll
                for (int i = 0; i < V; ++i) acc = op.combine(acc, op.lift(r[i], begin + k * V + i, ctx));
            }
            // Ragged end of the range (fewer than V elements).
            for (int64_t r = begin + nvec * V + lane; r < end; r += G) acc = op.combine(acc, op.lift(p[r], r, ctx));
        }
        acc = wave_fold(op, acc);
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

// Contiguous outputs ("columns"), one strided reduced dimension. `rstride` is that stride and
// `inner` the length of the contiguous run of outputs (the innermost kept dimension); a.kept
// holds the remaining, outer kept dimensions. VEC: every row of every column tile starts 16-byte
// aligned.
template <class Op, class Sink, bool VEC>
__global__ void __launch_bounds__(kBlock)
    reduce_cols_kernel(ReduceArgs a, int64_t rstride, int64_t inner, Op op, Sink sink) {
    using T = typename Op::In;
    using Acc = typename Op::Acc;
    constexpr int V = VEC ? 16 / static_cast<int>(sizeof(T)) : 1;
    constexpr int kWaves = kBlock / kWave;
    constexpr int U = 4;
    __shared__ Acc lds[kWaves - 1][kWave * V];
    const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
    const int64_t split = blockIdx.y;
    const int64_t begin = split * a.chunk;
    const int64_t end = begin + a.chunk < a.nred ? begin + a.chunk : a.nred;
    const int64_t tiles_inner = (inner + kWave * V - 1) / (kWave * V);
    const int64_t tiles = tiles_inner * (a.nout / inner);
    for (int64_t tile = blockIdx.x; tile < tiles; tile += gridDim.x) {
        const int64_t outer = tile / tiles_inner;
        const int64_t col = (tile - outer * tiles_inner) * (kWave * V) + lane * V;  // within the run
        const int64_t obase = outer * inner;                                       // first output of the run
        const T *src = reinterpret_cast<const T *>(a.src) + a.kept.offset(outer);
        const int valid = inner - col >= V ? V : (inner > col ? static_cast<int>(inner - col) : 0);
        Acc acc[V];
        typename Op::Ctx ctx[V];
#pragma unroll
        for (int i = 0; i < V; ++i) {
            acc[i] = op.init();
            ctx[i] = op.context(i < valid ? obase + col + i : 0);
        }
        if (valid == V) {
            int64_t r = begin + wave;
            for (; r + (U - 1) * kWaves < end; r += U * kWaves) {
                T t[U][V];
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    load_tile<T, V>(reinterpret_cast<const char *>(src + (r + u * kWaves) * rstride + col), t[u]);
                }
#pragma unroll
                for (int u = 0; u < U; ++u) {
#pragma unroll
                    for (int i = 0; i < V; ++i) acc[i] = op.combine(acc[i], op.lift(t[u][i], r + u * kWaves, ctx[i]));
                }
            }
            for (; r < end; r += kWaves) {
                T t[V];
                load_tile<T, V>(reinterpret_cast<const char *>(src + r * rstride + col), t);
#pragma unroll
                for (int i = 0; i < V; ++i) acc[i] = op.combine(acc[i], op.lift(t[i], r, ctx[i]));
            }
        } else if (valid > 0) {
            for (int64_t r = begin + wave; r < end; r += kWaves) {
#pragma unroll
                for (int i = 0; i < V; ++i) {
                    if (i < valid) acc[i] = op.combine(acc[i], op.lift(src[r * rstride + col + i], r, ctx[i]));
                }
            }
        }
        // Waves 1..3 hand their accumulators to wave 0, which folds them in wave order.
        __syncthreads();
        if (wave > 0) {
#pragma unroll
            for (int i = 0; i < V; ++i) lds[wave - 1][lane * V + i] = acc[i];
        }
        __syncthreads();
        if (wave == 0) {
#pragma unroll
            for (int i = 0; i < V; ++i) {
#pragma unroll
                for (int w = 0; w < kWaves - 1; ++w) acc[i] = op.combine(acc[i], lds[w][lane * V + i]);
                if (i < valid) {
                    if (a.splits > 1) put_partial(a.partials, a.nout, split, obase + col + i, acc[i]);
                    else sink.put(obase + col + i, acc[i], a.nred);
                }
            }
        }
    }
}

}  // namespace hmr
