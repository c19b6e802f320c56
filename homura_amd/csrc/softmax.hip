// hmr_softmax / hmr_softmax_workspace / hmr_test_softmax_plan
// (ref: csrc/homura_rocm.h:338-351, csrc/reduce.hip:162-360, 519-580).
//
// What is computed is cpu::softmax (ref: src/backend/cpu/misc.rs:15-51): per row,
//   max = fold(-inf, v > m ? v : m)      (a NaN never replaces)
//   sum = sum_k exp(x_k - max)
//   out = exp(x_k - max) / sum           or   x_k - max - ln(sum)
// in f64, rounded to the dtype. The consequences the CPU has are kept because the same
// expressions are evaluated: a row holding a NaN, holding +inf, or made of -inf only comes out
// all NaN; -inf entries give exactly 0 (softmax) or -inf (log_softmax).
//
// Precision per dtype (the result must land within one ulp of the dtype of the CPU's):
//   F16/BF16  f32 evaluation of exp (one f32 ulp is 2^-13 / 2^-16 of an output ulp); the row sum
//             is accumulated in f64.
//   F32       exp evaluated in f64 by a degree-11 polynomial after Cody-Waite reduction
//             (relative error < 2^-45, far inside an f32 ulp), f64 sum, one f64 reciprocal per row
//             instead of a division per element.
//   F64       the device library's exp and a true f64 division.
//
// Plans:
//   registers  contiguous rows up to 64*G*... elements: G lanes (one wave, a 256-lane or a
//              1024-lane workgroup) read the row once with 128-bit loads, keep it in registers
//              through all three phases and write it once. Algorithmic traffic only.
//   streaming  anything else (strided rows, rows too long for the register file): G lanes walk
//              the row three times (max, sum, write) with scalar loads.
// Rows are never cut across workgroups, so no workspace is needed (hmr_softmax_workspace: 0).
#include <cmath>

#include "dispatch.hpp"
#include "lines.hpp"
#include "reduce.hpp"

namespace hmr {
namespace {

// ---- exp in the evaluation type ------------------------------------------------------------------

// exp(t) for t <= 0 (or NaN) in f64, without a branch. |relative error| < 2^-36: an f32 result
// computed from it differs from the correctly rounded one only within 2^-12 ulp of a rounding boundary.
// Below -708 (where exp underflows; -inf included) the arithmetic runs on meaningless values, which the
// final select replaces by 0; a NaN propagates through every step.
//
// The Horner steps are written as the instruction itself with the coefficient in a scalar register pair:
// left to the compiler each step becomes a register copy of the coefficient plus a two-address v_fmac_f64.
__device__ __forceinline__ double horner_step(double p, double r, double coefficient) {
    double out;
    asm("v_fma_f64 %0, %1, %2, %3" : "=v"(out) : "v"(p), "v"(r), "s"(coefficient));
    return out;
}

// `dead`: the caller does not want this lane's value (it gets 0).
__device__ __forceinline__ double exp_neg_f64(double t, bool dead = false) {
    const double kLog2e = 1.4426950408889634074;
    const double kLn2Hi = 6.93147180369123816490e-01;
    const double kLn2Lo = 1.90821492927058770002e-10;
    double n = rint(t * kLog2e);
    double r = fma(-n, kLn2Hi, t);
    r = fma(-n, kLn2Lo, r);  // |r| <= 0.3466
    // Taylor to degree 9: remainder < 0.3466^10 / 10! < 2^-37.
    double p = horner_step(1.0 / 362880.0, r, 1.0 / 40320.0);
    p = horner_step(p, r, 1.0 / 5040.0);
    p = horner_step(p, r, 1.0 / 720.0);
    p = horner_step(p, r, 1.0 / 120.0);
    p = horner_step(p, r, 1.0 / 24.0);
    p = horner_step(p, r, 1.0 / 6.0);
    p = fma(p, r, 0.5);
    p = fma(p, r, 1.0);
    p = fma(p, r, 1.0);
    // Scale by 2^n, n in [-1022, 0].
    p = ldexp(p, static_cast<int>(n));
    return (t < -708.0 || dead) ? 0.0 : p;
}

template <class T>
struct SoftmaxMath;

constexpr float kLog2eF = 1.44269504088896340736f;

// Halves: values travel as f32. Anything whose relative error stays near 2^-17 lands within one ulp
// of an 8- or 11-bit result, so the exponentials come from the hardware's 2^x (v_exp_f32, 1 ulp):
//   for the sum   2^((x - max) log2 e)              (results below 2^-126 may flush: they are
//                                                    below 2^-126 of a sum that is at least 1)
//   for the output 2^((x - max) log2 e - log2 sum)  evaluated as ldexp(2^(.. + 64), -64), which keeps
//                                                    subnormal results (v_exp_f32 alone flushes them).
// The output form is evaluated per element in the last phase instead of keeping every exponential
// in registers, which lets a lane hold 128 packed elements of its row.
template <class T>
struct HalfMath {
    using X = float;  // a row element in registers
    using E = float;  // exp(x - max), and the per-row scale
    static constexpr bool kKeep = false;
    static __device__ __forceinline__ X load(T v) { return Comp<T>::up(v); }
    static __device__ __forceinline__ void unpack(const u32x4 &r, X (&x)[8]) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            if constexpr (std::is_same_v<T, bf16_t>) {
                x[2 * j] = __uint_as_float(r[j] << 16);
                x[2 * j + 1] = __uint_as_float(r[j] & 0xFFFF0000u);
            } else {
                x[2 * j] = f16_widen(f16_t{static_cast<uint16_t>(r[j] & 0xFFFFu)});
                x[2 * j + 1] = f16_widen(f16_t{static_cast<uint16_t>(r[j] >> 16)});
            }
        }
    }
    // Results in the evaluation type -> a packed chunk of the row.
    static __device__ __forceinline__ u32x4 pack(const float (&y)[8]) {
        u32x4 r;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            if constexpr (std::is_same_v<T, bf16_t>) {
                r[j] = bf16_round_pair(y[2 * j], y[2 * j + 1]);
            } else {
                r[j] = static_cast<uint32_t>(f16_round(y[2 * j]).bits) | (static_cast<uint32_t>(f16_round(y[2 * j + 1]).bits) << 16);
            }
        }
        return r;
    }
    static __device__ __forceinline__ E ex(X x, X mx) { return __builtin_amdgcn_exp2f((x - mx) * kLog2eF); }
    static __device__ __forceinline__ double wide(E e) { return static_cast<double>(e); }
    static __device__ __forceinline__ E scale(double sum) { return 64.0f - __builtin_log2f(static_cast<float>(sum)); }
    static __device__ __forceinline__ E lg(double sum) { return static_cast<float>(log(sum)); }
    static __device__ __forceinline__ float soft(X x, X mx, E, E bias) {  // bias = 64 - log2 sum
        return __builtin_ldexpf(__builtin_amdgcn_exp2f(__builtin_fmaf(x - mx, kLog2eF, bias)), -64);
    }
    static __device__ __forceinline__ float logsoft(X x, X mx, E log_sum) { return x - mx - log_sum; }
    static __device__ __forceinline__ T down(float y) { return Comp<T>::down(y); }
};
template <>
struct SoftmaxMath<f16_t> : HalfMath<f16_t> {};
template <>
struct SoftmaxMath<bf16_t> : HalfMath<bf16_t> {};

template <>
struct SoftmaxMath<float> {
    using X = float;
    using E = double;
    static constexpr bool kKeep = true;  // the f64 exponentials stay in registers for the last phase
    static __device__ __forceinline__ X load(float v) { return v; }
    static __device__ __forceinline__ void unpack(const u32x4 &r, X (&x)[4]) {
#pragma unroll
        for (int i = 0; i < 4; ++i) x[i] = __uint_as_float(r[i]);
    }
    static __device__ __forceinline__ E ex(X x, X mx, bool dead = false) {
        return exp_neg_f64(static_cast<double>(x) - static_cast<double>(mx), dead);
    }
    static __device__ __forceinline__ double wide(E e) { return e; }
    static __device__ __forceinline__ E scale(double sum) { return 1.0 / sum; }
    static __device__ __forceinline__ E lg(double sum) { return log(sum); }
    static __device__ __forceinline__ float soft(X, X, E e, E inv_sum) { return static_cast<float>(e * inv_sum); }
    static __device__ __forceinline__ float logsoft(X x, X mx, E log_sum) {
        return static_cast<float>(static_cast<double>(x) - static_cast<double>(mx) - log_sum);
    }
    static __device__ __forceinline__ float down(float y) { return y; }
    static __device__ __forceinline__ u32x4 pack(const float (&y)[4]) {
        return u32x4{__float_as_uint(y[0]), __float_as_uint(y[1]), __float_as_uint(y[2]), __float_as_uint(y[3])};
    }
};

template <>
struct SoftmaxMath<double> {
    using X = double;
    using E = double;
    static constexpr bool kKeep = true;
    static __device__ __forceinline__ X load(double v) { return v; }
    static __device__ __forceinline__ void unpack(const u32x4 &r, X (&x)[2]) {
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            x[i] = __longlong_as_double(static_cast<int64_t>(static_cast<uint64_t>(r[2 * i]) |
                                                             (static_cast<uint64_t>(r[2 * i + 1]) << 32)));
        }
    }
    static __device__ __forceinline__ E ex(X x, X mx, bool dead = false) { return dead ? 0.0 : exp(x - mx); }
    static __device__ __forceinline__ double wide(E e) { return e; }
    static __device__ __forceinline__ E scale(double sum) { return sum; }
    static __device__ __forceinline__ E lg(double sum) { return log(sum); }
    static __device__ __forceinline__ double soft(X, X, E e, E sum) { return e / sum; }
    static __device__ __forceinline__ double logsoft(X x, X mx, E log_sum) { return x - mx - log_sum; }
    static __device__ __forceinline__ double down(double y) { return y; }
    static __device__ __forceinline__ u32x4 pack(const double (&y)[2]) {
        u32x4 r;
        __builtin_memcpy(&r, y, 16);
        return r;
    }
};

// max(m, a, b) in one instruction. How a NaN operand is treated does not matter to softmax: a row
// holding a NaN comes out all NaN whatever its max is taken to be.
__device__ __forceinline__ float max3(float m, float a, float b) {
    float r;
    asm("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(m), "v"(a), "v"(b));
    return r;
}
__device__ __forceinline__ double max3(double m, double a, double b) {
    m = a > m ? a : m;
    return b > m ? b : m;
}

// ---- combining across the lanes of a row ---------------------------------------------------------

struct MaxOp {
    static constexpr bool kCommutative = true;
    using Acc = double;
    __device__ __forceinline__ Acc combine(Acc a, Acc b) const { return b > a ? b : a; }
};
struct MaxOpF {
    static constexpr bool kCommutative = true;
    using Acc = float;
    __device__ __forceinline__ Acc combine(Acc a, Acc b) const { return b > a ? b : a; }
};
struct SumOp {
    static constexpr bool kCommutative = true;  // IEEE addition is
    using Acc = double;
    __device__ __forceinline__ Acc combine(Acc a, Acc b) const { return a + b; }
};

// Folds `v` over the G lanes that share a row: one wave, or G / 64 neighbouring waves of the workgroup
// that meet in LDS (`lds` has one slot per wave of the workgroup).
template <int G, class Op>
__device__ __forceinline__ typename Op::Acc row_fold(const Op &op, typename Op::Acc v, typename Op::Acc *lds) {
    v = wave_fold(op, v);
    if constexpr (G > kWave) {
        constexpr int kWaves = G / kWave;
        const int first = static_cast<int>(threadIdx.x) / G * kWaves;
        __syncthreads();
        if (threadIdx.x % kWave == 0) lds[threadIdx.x / kWave] = v;
        __syncthreads();
        v = lds[first];
#pragma unroll
        for (int w = 1; w < kWaves; ++w) v = op.combine(v, lds[first + w]);
    }
    return v;
}

struct SoftmaxArgs {
    char *out;        // element (0,..) of the output rows
    const char *src;  // element (0,..) of the source rows
    Walk out_rows;    // row index -> output offset
    Walk src_rows;    // row index -> source offset
    int64_t nrows;
    int64_t n;
    int64_t so, si;
    int32_t stream_stores;  // registers plan: nontemporal stores instead of write-through ones
};

// Contiguous rows held in registers, as loaded (16-byte chunks). G lanes per row, each with C
// chunks of V elements: chunk c of lane l covers elements (c*G + l)*V .. +V, so every load of the
// group is one contiguous, coalesced span. Rows are whole chunks (n is a multiple of V).
//
// All C loads of a lane are issued back to back and unconditionally: a branch between loads would
// make each wait for the one before. A chunk past the row's end re-reads the row's last chunk, which
// cannot change the max, and is left out of the sum and of the stores.
//
// WALK = false: the rows form one dimension (row r starts r * stride elements in), which is what a
// contiguous tensor gives; WALK = true: up to 25 row dimensions, decoded per row.
// Stores write through the compute die's L2 (see OutStores in map.hpp), or are nontemporal for outputs far larger
// than the memory-side cache (`stream_stores`).
template <class T, int G, int C, bool LOG, bool WALK>
__global__ void __launch_bounds__(G > kBlock ? G : kBlock) softmax_regs_kernel(SoftmaxArgs a) {
    using M = SoftmaxMath<T>;
    using X = typename M::X;
    using E = typename M::E;
    using MaxFold = std::conditional_t<std::is_same_v<X, float>, MaxOpF, MaxOp>;
    constexpr int V = 16 / static_cast<int>(sizeof(T));
    constexpr int kThreads = G > kBlock ? G : kBlock;
    constexpr int kRowsPerBlock = kThreads / G;
    constexpr bool kKeep = M::kKeep && !LOG;
    __shared__ double lds[kThreads / kWave];
    const int lane = threadIdx.x % G;
    const int64_t groups = (a.nrows + kRowsPerBlock - 1) / kRowsPerBlock;
    const int nvec = static_cast<int>(a.n / V);  // chunks in a row (>= 1)
    for (int64_t g = blockIdx.x; g < groups; g += gridDim.x) {
        // A row belongs to whole waves (G is a multiple of 64): its number is the same in every lane of one.
        const int64_t row = g * kRowsPerBlock + __builtin_amdgcn_readfirstlane(static_cast<int>(threadIdx.x) / G);
        const bool live = row < a.nrows;
        const int64_t r = live ? row : a.nrows - 1;  // idle lanes of the last group redo the last row, without storing
        const T *src = reinterpret_cast<const T *>(a.src) + (WALK ? a.src_rows.offset(r) : r * a.src_rows.stride[0]);
        T *out = reinterpret_cast<T *>(a.out) + (WALK ? a.out_rows.offset(r) : r * a.out_rows.stride[0]);
        const __amdgpu_buffer_rsrc_t out_row = __builtin_amdgcn_make_buffer_rsrc(out, 0, -1, 0x00020000);
        // Phase 0: one pass over memory.
        u32x4 raw[C];
#pragma unroll
        for (int c = 0; c < C; ++c) {
            // A uniform row pointer plus a 32-bit byte offset per lane: one address register per chunk.
            const uint32_t tile = static_cast<uint32_t>(c * G + lane);
            const uint32_t t = tile < static_cast<uint32_t>(nvec) ? tile : static_cast<uint32_t>(nvec - 1);
            const u32x4 *q = reinterpret_cast<const u32x4 *>(reinterpret_cast<const char *>(src) + t * 16u);
            if constexpr (kStreamLoads) raw[c] = __builtin_nontemporal_load(q);
            else raw[c] = *q;
        }
        __builtin_amdgcn_sched_barrier(0);  // every load is out before anything waits for one
        // Phase 1: max.
        X mx = -__builtin_huge_valf();
#pragma unroll
        for (int c = 0; c < C; ++c) {
            X x[V];
            M::unpack(raw[c], x);
#pragma unroll
            for (int i = 0; i < V; i += 2) mx = max3(mx, x[i], x[i + 1]);
        }
        mx = row_fold<G>(MaxFold{}, mx, reinterpret_cast<X *>(lds));
        // Phase 2: exponentials and their f64 sum.
        double sum = 0.0;
        E ex[kKeep ? C : 1][kKeep ? V : 1];  // chunk c is defined where did[c]
        bool did[C];
#pragma unroll
        for (int c = 0; c < C; ++c) {
            X x[V];
            forget(raw[c]);
            M::unpack(raw[c], x);
            const bool inside = c * G + lane < nvec;
            if constexpr (std::is_same_v<E, double>) {
                // An f64 exponential is some twenty-five instructions. When no lane of the wave holds an
                // element of this chunk within 708 of the max (a masked span of attention scores, a
                // chunk past the row's end), every exponential of the chunk is exactly 0: skip them all.
                bool some = false;
#pragma unroll
                for (int i = 0; i < V; ++i) some |= !(static_cast<double>(x[i]) - static_cast<double>(mx) < -708.0);
                did[c] = __builtin_amdgcn_ballot_w64(some && inside) != 0;
                if (did[c]) {
#pragma unroll
                    for (int i = 0; i < V; ++i) {
                        const double v = M::ex(x[i], mx, !inside);
                        sum += v;
                        if constexpr (kKeep) ex[c][i] = v;
                    }
                }
            } else {
                // Eight f32 terms pairwise (relative error ~2^-22), then one f64 addition per chunk.
                if (inside) {
                    E e[V];
#pragma unroll
                    for (int i = 0; i < V; ++i) e[i] = M::ex(x[i], mx);
                    float part = ((e[0] + e[1]) + (e[2] + e[3])) + ((e[4] + e[5]) + (e[6] + e[7]));
                    if constexpr (LOG) {
                        // log_softmax of a row that one element dominates is -log(1 + s) ~ -s with s the sum of
                        // the other terms, and s must keep its own relative accuracy: next to a 1 in an f32 sum
                        // it would keep 2^-24 absolute. The terms that are exactly 1 (the maximum and anything
                        // that rounds to it) are counted instead of added; the count joins the f64 sum. Only a
                        // chunk whose terms reach 1 together can hold one: the few that do are summed again.
                        if (part >= 1.0f) {
                            float ones = 0.0f;
#pragma unroll
                            for (int i = 0; i < V; ++i) {
                                const bool one = e[i] == 1.0f;
                                ones += one ? 1.0f : 0.0f;
                                e[i] = one ? 0.0f : e[i];
                            }
                            part = ((e[0] + e[1]) + (e[2] + e[3])) + ((e[4] + e[5]) + (e[6] + e[7]));
                            sum += static_cast<double>(ones);
                        }
                    }
                    sum += static_cast<double>(part);
                }
            }
            // One chunk at a time: interleaving the chunks' independent chains would multiply the live
            // temporaries.
            __builtin_amdgcn_sched_barrier(0);
        }
        sum = row_fold<G>(SumOp{}, sum, lds);
        // Phase 3: write once.
        const E scale = LOG ? M::lg(sum) : M::scale(sum);
#pragma unroll
        for (int c = 0; c < C; ++c) {
            const int tile = c * G + lane;
            X x[V];
            forget(raw[c]);
            M::unpack(raw[c], x);
            decltype(M::logsoft(x[0], mx, scale)) res[V];
#pragma unroll
            for (int i = 0; i < V; ++i) {
                if constexpr (LOG) {
                    res[i] = M::logsoft(x[i], mx, scale);
                } else if constexpr (kKeep) {
                    // A skipped chunk holds exact zeros: 0 * scale, which is 0 unless the row's sum is NaN.
                    res[i] = M::soft(x[i], mx, E(0), scale);
                    if (did[c]) res[i] = M::soft(x[i], mx, ex[c][i], scale);
                } else {
                    res[i] = M::soft(x[i], mx, E(0), scale);
                }
            }
            if (live && tile < nvec) {
                if (a.stream_stores) {
                    __builtin_nontemporal_store(M::pack(res), reinterpret_cast<u32x4 *>(reinterpret_cast<char *>(out) + static_cast<uint32_t>(tile) * 16u));
                } else {
                    __builtin_amdgcn_raw_buffer_store_b128(M::pack(res), out_row, tile * 16, 0, 17 /* sc0 sc1 */);
                }
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    }
}

// Any layout: G lanes walk the row three times.
template <class T, int G, bool LOG>
__global__ void __launch_bounds__(kBlock) softmax_stream_kernel(SoftmaxArgs a) {
    using M = SoftmaxMath<T>;
    using X = typename M::X;
    using E = typename M::E;
    using MaxFold = std::conditional_t<std::is_same_v<X, float>, MaxOpF, MaxOp>;
    constexpr int kRowsPerBlock = kBlock / G;
    __shared__ double lds[kBlock / kWave];
    const int lane = threadIdx.x % G;
    const int64_t groups = (a.nrows + kRowsPerBlock - 1) / kRowsPerBlock;
    for (int64_t g = blockIdx.x; g < groups; g += gridDim.x) {
        const int64_t row = g * kRowsPerBlock + threadIdx.x / G;
        const bool live = row < a.nrows;
        const T *src = reinterpret_cast<const T *>(a.src) + (live ? a.src_rows.offset(row) : 0);
        T *out = reinterpret_cast<T *>(a.out) + (live ? a.out_rows.offset(row) : 0);
        const int64_t n = live ? a.n : 0;
        X mx = -__builtin_huge_valf();
        for (int64_t k = lane; k < n; k += G) {
            X v = M::load(src[k * a.si]);
            mx = v > mx ? v : mx;
        }
        mx = row_fold<G>(MaxFold{}, mx, reinterpret_cast<X *>(lds));
        double sum = 0.0;
        for (int64_t k = lane; k < n; k += G) sum += M::wide(M::ex(M::load(src[k * a.si]), mx));
        sum = row_fold<G>(SumOp{}, sum, lds);
        const E scale = LOG ? M::lg(sum) : M::scale(sum);
        for (int64_t k = lane; k < n; k += G) {
            X v = M::load(src[k * a.si]);
            if constexpr (LOG) out[k * a.so] = M::down(M::logsoft(v, mx, scale));
            else out[k * a.so] = M::down(M::soft(v, mx, M::kKeep ? M::ex(v, mx) : E(0), scale));
        }
    }
}

// ---- plan -----------------------------------------------------------------------------------------

struct SoftmaxPlan {
    bool regs = false;  // registers plan (else streaming)
    int group = kWave;  // lanes per row
    int tiles = 0;      // registers plan: 128-bit tiles per lane
};

// 128-bit chunks of the row a lane keeps: 8 (32 f32 or 16 f64 values, plus their f64 exponentials),
// or 16 packed chunks (128 values) of a 16-bit type, whose exponentials are not kept.
constexpr int max_tiles(int elem) { return elem == 2 ? 16 : 8; }

// The plan depends on the source only (sizes, strides, alignment), so that the size query, which
// does not see the output, agrees with the launch; the launch falls back to streaming by itself
// when the output is not laid out like a contiguous, aligned row.
SoftmaxPlan plan_softmax(const hmr_tensor_desc &src_rows, int64_t n, int64_t si, const Walk &ws) {
    SoftmaxPlan p;
    const int elem = dtype_size(src_rows.dtype);
    const int vec = 16 / elem;
    bool aligned = (n == 1 || si == 1) &&
                   reinterpret_cast<uintptr_t>(static_cast<char *>(src_rows.data) + src_rows.offset * elem) % 16 == 0;
    for (int d = 0; aligned && d < ws.ndim; ++d) aligned = (ws.stride[d] * elem) % 16 == 0;
    const int64_t tiles = (n + vec - 1) / vec;  // 128-bit tiles in a row
    if (aligned && n >= 16 && n % vec == 0) {
        // Lanes per row and chunks per lane, first fit. 16-bit rows stay packed (4 registers per chunk);
        // wider rows also keep their f64 exponentials (8 more registers per f32 chunk), so they spread over
        // two waves before a lane takes more than four chunks: more resident waves hide the row loads.
        struct Step {
            int group, tiles;
        };
        static const Step half_steps[] = {{kWave, 16}, {kBlock, 16}, {1024, 16}};
        static const Step wide_steps[] = {{kWave, 4}, {128, 4}, {kBlock, 8}, {1024, 8}};
        const Step *steps = elem == 2 ? half_steps : wide_steps;
        const int nsteps = elem == 2 ? 3 : 4;
        for (int k = 0; k < nsteps; ++k) {
            const int g = steps[k].group;
            const int64_t lim = steps[k].tiles;
            int64_t per = (tiles + g - 1) / g;
            if (per <= lim && per <= max_tiles(elem)) {
                p.regs = true;
                p.group = g;
                p.tiles = per <= 1 ? 1 : (per <= 2 ? 2 : (per <= 4 ? 4 : (per <= 8 ? 8 : 16)));
                return p;
            }
        }
    }
    p.regs = false;
    p.group = n <= 4096 ? kWave : kBlock;
    p.tiles = 0;
    return p;
}

template <class T, bool LOG>
void launch_softmax(const SoftmaxPlan &p, const SoftmaxArgs &a, bool out_ok, hipStream_t stream) {
    const int64_t cap = 1 << 20;
    auto blocks = [&](int rows_per_block) {
        int64_t b = (a.nrows + rows_per_block - 1) / rows_per_block;
        return dim3(static_cast<unsigned>(b < cap ? (b < 1 ? 1 : b) : cap));
    };
    if (p.regs && out_ok) {
        auto run = [&](auto g, auto c) {
            constexpr int G = decltype(g)::value, C = decltype(c)::value;
            constexpr int kThreads = G > kBlock ? G : kBlock;
            if (a.src_rows.ndim <= 1) {
                hipLaunchKernelGGL((softmax_regs_kernel<T, G, C, LOG, false>), blocks(kThreads / G), dim3(kThreads), 0, stream, a);
            } else {
                hipLaunchKernelGGL((softmax_regs_kernel<T, G, C, LOG, true>), blocks(kThreads / G), dim3(kThreads), 0, stream, a);
            }
        };
        auto with_tiles = [&](auto g) {
            switch (p.tiles) {
                case 1: run(g, IntTag<1>{}); break;
                case 2: run(g, IntTag<2>{}); break;
                case 4: run(g, IntTag<4>{}); break;
                case 8: run(g, IntTag<8>{}); break;
                default:
                    if constexpr (sizeof(T) == 2) run(g, IntTag<16>{});
                    break;
            }
        };
        if (p.group == kWave) with_tiles(IntTag<kWave>{});
        else if (p.group == 128) with_tiles(IntTag<128>{});
        else if (p.group == kBlock) with_tiles(IntTag<kBlock>{});
        else with_tiles(IntTag<1024>{});
        return;
    }
    const int group = p.regs ? (a.n <= 4096 ? kWave : kBlock) : p.group;
    if (group == kWave) {
        hipLaunchKernelGGL((softmax_stream_kernel<T, kWave, LOG>), blocks(kBlock / kWave), dim3(kBlock), 0, stream, a);
    } else {
        hipLaunchKernelGGL((softmax_stream_kernel<T, kBlock, LOG>), blocks(1), dim3(kBlock), 0, stream, a);
    }
}

}  // namespace
}  // namespace hmr

using hmr::fenced;

extern "C" {

hmr_status hmr_softmax_workspace(const hmr_tensor_desc *src_rows, int64_t n, int64_t src_stride, int64_t *bytes) {
    return fenced([&] {
        int64_t nrows = 0;
        if (hmr_status s = hmr::check_rows(*src_rows, *src_rows, n, 0, src_stride, nrows)) return s;
        *bytes = 0;  // no plan of this library cuts a row across workgroups
        return HMR_OK;
    });
}

hmr_status hmr_test_softmax_plan(const hmr_tensor_desc *src_rows, int64_t n, int64_t src_stride, int32_t *split,
                                 int32_t *group, int32_t *cache) {
    return fenced([&] {
        int64_t nrows = 0;
        if (hmr_status s = hmr::check_rows(*src_rows, *src_rows, n, 0, src_stride, nrows)) return s;
        hmr::Walk wo, ws;
        hmr::walk_pair(*src_rows, *src_rows, wo, ws);
        hmr::SoftmaxPlan p = hmr::plan_softmax(*src_rows, n, src_stride, ws);
        *split = 0;
        *group = p.group;
        *cache = p.regs ? p.tiles * (16 / hmr::dtype_size(src_rows->dtype)) : 0;
        return HMR_OK;
    });
}

hmr_status hmr_softmax(hmr_context_t ctx, const hmr_tensor_desc *out_rows, const hmr_tensor_desc *src_rows, int64_t n,
                       int64_t out_stride, int64_t src_stride, int32_t log, void *workspace,
                       int64_t workspace_bytes) {
    (void)workspace;
    (void)workspace_bytes;
    return fenced([&] {
        int64_t nrows = 0;
        if (hmr_status s = hmr::check_rows(*out_rows, *src_rows, n, out_stride, src_stride, nrows)) return s;
        if (nrows == 0 || n == 0) return HMR_OK;
        hmr::SoftmaxArgs a{};
        const int elem = hmr::dtype_size(src_rows->dtype);
        a.out = static_cast<char *>(out_rows->data) + out_rows->offset * elem;
        a.src = static_cast<const char *>(src_rows->data) + src_rows->offset * elem;
        a.nrows = hmr::walk_pair(*out_rows, *src_rows, a.out_rows, a.src_rows);
        a.n = n;
        a.so = out_stride;
        a.si = src_stride;
        a.stream_stores = a.nrows * n * elem >= hmr::kStreamStoreBytes ? 1 : 0;
        hmr::SoftmaxPlan plan = hmr::plan_softmax(*src_rows, n, src_stride, a.src_rows);
        bool out_ok = (n == 1 || out_stride == 1) && reinterpret_cast<uintptr_t>(a.out) % 16 == 0;
        for (int d = 0; out_ok && d < a.out_rows.ndim; ++d) out_ok = (a.out_rows.stride[d] * elem) % 16 == 0;
        return hmr::queue_on(ctx, "softmax", [&](hipStream_t stream) {
            if (out_rows->dtype != src_rows->dtype) return false;
            return hmr::with_float_type(out_rows->dtype, [&](auto t) {
                using T = typename decltype(t)::type;
                if (log != 0) hmr::launch_softmax<T, true>(plan, a, out_ok, stream);
                else hmr::launch_softmax<T, false>(plan, a, out_ok, stream);
            });
        });
    });
}

}  // extern "C"
