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
    // The logarithm of a row's sum (1 <= sum, the maximum's own term being 1), for results that are rounded to 8
    // or 11 bits: f32 arithmetic serves and costs a dozen registers less than the f64 routine, which the rows held
    // in registers cannot spare. Just above 1 (a row that one element dominates) log(1 + t) must keep the
    // accuracy of t, which 1 + t in f32 has lost: the series there (t < 2^-6: the next term is below 2^-32 of t),
    // the hardware's log2 elsewhere (relative error below 2^-17 of a logarithm that is at least 2^-6).
    static __device__ __forceinline__ E lg(double sum) {
        const float t = static_cast<float>(sum - 1.0);
        const float series = t * (1.0f + t * (-0.5f + t * (0.333333343f + t * (-0.25f + t * 0.2f))));
        const float general = __builtin_amdgcn_logf(static_cast<float>(sum)) * 0.693147182f;
        return t < 0.015625f ? series : general;  // a NaN sum takes the second and stays NaN
    }
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

// A value that every lane of the wave holds alike, moved to scalar registers: it stops costing a vector register
// for as long as it lives (a row's maximum, sum and scale live across whole phases).
template <class A>
__device__ __forceinline__ A uniform(A v) {
    constexpr int words = static_cast<int>(sizeof(A)) / 4;
    static_assert(sizeof(A) % 4 == 0, "whole words");
    uint32_t w[words];
    __builtin_memcpy(w, &v, sizeof(A));
#pragma unroll
    for (int i = 0; i < words; ++i) w[i] = static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(static_cast<int>(w[i])));
    __builtin_memcpy(&v, w, sizeof(A));
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
//
// log_softmax waits for one f64 logarithm per row - a chain of dependent instructions that a compute unit can only
// hide behind another workgroup. The 1024-lane form of a 16-bit row with up to four chunks a lane is therefore held
// to 64 registers (the softmax form needs 60 by itself), so that two workgroups share a compute unit: a
// [4096, 32000] bf16 log_softmax 123 -> 93 us.
template <class T, int G, int C, bool LOG, bool WALK>
__global__ void __launch_bounds__(G > kBlock ? G : kBlock, (LOG && G == 1024 && C <= 4 && sizeof(T) == 2) ? 8 : 1) softmax_regs_kernel(SoftmaxArgs a) {
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
        // Phase 0: one pass over memory. The lane number is made opaque here and again before the stores: what is
        // derived from it (a chunk's offset, whether it lies inside the row) is then computed where it is used, a few
        // instructions per chunk, instead of being hoisted out of the loop over rows and kept - two registers per
        // chunk, which cost the sixteen-chunk form a workgroup per compute unit.
        int at = lane;
        asm volatile("" : "+v"(at));
        u32x4 raw[C];
#pragma unroll
        for (int c = 0; c < C; ++c) {
            // A uniform row pointer plus a 32-bit byte offset per lane: one address register per chunk.
            const uint32_t tile = static_cast<uint32_t>(c * G + at);
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
            __builtin_amdgcn_sched_barrier(0);  // a chunk at a time: unpacked ahead, the row would fill the registers
        }
        mx = uniform(row_fold<G>(MaxFold{}, mx, reinterpret_cast<X *>(lds)));  // a row is whole waves
        // Phase 2: exponentials and their f64 sum.
        double sum = 0.0;
        E ex[kKeep ? C : 1][kKeep ? V : 1];  // chunk c is defined where did[c]
        bool did[C];
#pragma unroll
        for (int c = 0; c < C; ++c) {
            X x[V];
            forget(raw[c]);
            M::unpack(raw[c], x);
            const bool inside = c * G + at < nvec;
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
        sum = uniform(row_fold<G>(SumOp{}, sum, lds));
        // Phase 3: write once.
        E scale;
        if constexpr (LOG && G > kBlock) {
            // The logarithm is an f64 routine of some hundred instructions, the same for the whole row: with
            // sixteen waves on a row one of them evaluates it and the others take it from LDS.
            __shared__ E row_scale;
            if (threadIdx.x < kWave) {
                const E v = M::lg(sum);
                if (threadIdx.x == 0) row_scale = v;
            }
            __syncthreads();
            scale = uniform(row_scale);
        } else {
            scale = uniform(LOG ? M::lg(sum) : M::scale(sum));
        }
        asm volatile("" : "+v"(at));
#pragma unroll
        for (int c = 0; c < C; ++c) {
            const int tile = c * G + at;
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

// ---- few long rows: a row cut across workgroups ----------------------------------------------------------
//
// A contiguous row too long for the registers of one workgroup, or so few rows that a workgroup per row leaves
// most of the GPU idle, is cut into slices of C chunks per lane of a 256-lane workgroup. Two launches
// (ref: csrc/reduce.hip:314-360 plans the same split): the first leaves every slice's maximum and the sum of
// its exponentials about that maximum in the workspace; the second folds a row's slices - in slice order, so
// the result does not depend on which workgroup ran when - into the row's maximum and sum, and writes its own
// slice. A slice made of -inf only contributes nothing (and a row made of nothing else comes out NaN, as on
// the CPU). KEEP: the first launch reads through the caches, so that the second finds a source of up to a
// couple of hundred megabytes in the memory-side cache; larger sources stream both times.
// exp(t), t <= 0, for moving a sum of exponentials to a higher maximum: to the accuracy the sums themselves have
// (F64 rows: the library's exp; everything else is judged in f32 or less, and the polynomial's 2^-36 is plenty).
template <class X>
__device__ __forceinline__ double rescale(double t) {
    if constexpr (std::is_same_v<X, double>) return exp(t);
    else return exp_neg_f64(t);
}

struct SlicePartial {
    double max, sum;
};

struct SliceArgs {
    char *out;
    const char *src;
    Walk out_rows, src_rows;
    int64_t nrows, n;
    int64_t slices;  // per row
    SlicePartial *partials;  // [row][slice]
    int32_t stream_stores;
};

// exp(x - mx) summed over the V elements of one chunk, as the registers kernel sums them.
template <class T, bool LOG>
__device__ __forceinline__ double chunk_sum(const u32x4 &raw, typename SoftmaxMath<T>::X mx) {
    using M = SoftmaxMath<T>;
    using X = typename M::X;
    using E = typename M::E;
    constexpr int V = 16 / static_cast<int>(sizeof(T));
    X x[V];
    M::unpack(raw, x);
    // An element of -inf adds nothing, also about a maximum of -inf (where exp(-inf + inf) would say NaN): a
    // part of a row may be -inf throughout while the row is not. A NaN adds itself whatever the maximum.
    const X low = -__builtin_huge_valf();
    if constexpr (std::is_same_v<E, double>) {
        double sum = 0.0;
#pragma unroll
        for (int i = 0; i < V; ++i) sum += x[i] == low ? 0.0 : M::ex(x[i], mx);
        return sum;
    } else {
        E e[V];
#pragma unroll
        for (int i = 0; i < V; ++i) e[i] = x[i] == low ? 0.0f : M::ex(x[i], mx);
        float part = ((e[0] + e[1]) + (e[2] + e[3])) + ((e[4] + e[5]) + (e[6] + e[7]));
        double sum = 0.0;
        if constexpr (LOG) {
            // The terms that are exactly 1 are counted, not added (see the registers kernel).
            if (part >= 1.0f) {
                float ones = 0.0f;
#pragma unroll
                for (int i = 0; i < V; ++i) {
                    const bool one = e[i] == 1.0f;
                    ones += one ? 1.0f : 0.0f;
                    e[i] = one ? 0.0f : e[i];
                }
                part = ((e[0] + e[1]) + (e[2] + e[3])) + ((e[4] + e[5]) + (e[6] + e[7]));
                sum = static_cast<double>(ones);
            }
        }
        return sum + static_cast<double>(part);
    }
}

template <class T, int C, bool LOG, bool KEEP>
__global__ void __launch_bounds__(kBlock) softmax_slice_stats_kernel(SliceArgs a) {
    using M = SoftmaxMath<T>;
    using X = typename M::X;
    using MaxFold = std::conditional_t<std::is_same_v<X, float>, MaxOpF, MaxOp>;
    constexpr int V = 16 / static_cast<int>(sizeof(T));
    __shared__ double lds[kBlock / kWave];
    const int64_t row = blockIdx.x / a.slices, slice = blockIdx.x - row * a.slices;
    const int lane = threadIdx.x;
    const int64_t nvec = a.n / V, first = slice * (C * kBlock);
    const char *src = a.src + a.src_rows.offset(row) * static_cast<int64_t>(sizeof(T));
    u32x4 raw[C];
    bool inside[C];
#pragma unroll
    for (int c = 0; c < C; ++c) {
        const int64_t tile = first + c * kBlock + lane;
        inside[c] = tile < nvec;
        const u32x4 *q = reinterpret_cast<const u32x4 *>(src + (inside[c] ? tile : nvec - 1) * 16);
        if constexpr (KEEP) raw[c] = *q;
        else raw[c] = __builtin_nontemporal_load(q);
    }
    __builtin_amdgcn_sched_barrier(0);
    X mx = -__builtin_huge_valf();
#pragma unroll
    for (int c = 0; c < C; ++c) {
        X x[V];
        M::unpack(raw[c], x);
        X m = -__builtin_huge_valf();
#pragma unroll
        for (int i = 0; i < V; i += 2) m = max3(m, x[i], x[i + 1]);
        mx = inside[c] && m > mx ? m : mx;
    }
    mx = row_fold<kBlock>(MaxFold{}, mx, reinterpret_cast<X *>(lds));
    double sum = 0.0;
#pragma unroll
    for (int c = 0; c < C; ++c) {
        forget(raw[c]);
        const double part = chunk_sum<T, LOG>(raw[c], mx);
        sum += inside[c] ? part : 0.0;
    }
    sum = row_fold<kBlock>(SumOp{}, sum, lds);
    if (lane == 0) a.partials[blockIdx.x] = SlicePartial{static_cast<double>(mx), sum};
}

template <class T, int C, bool LOG>
__global__ void __launch_bounds__(kBlock) softmax_slice_write_kernel(SliceArgs a) {
    using M = SoftmaxMath<T>;
    using X = typename M::X;
    using E = typename M::E;
    constexpr int V = 16 / static_cast<int>(sizeof(T));
    __shared__ double lds[kBlock / kWave];
    const int64_t row = blockIdx.x / a.slices, slice = blockIdx.x - row * a.slices;
    const int lane = threadIdx.x;
    const int64_t nvec = a.n / V, first = slice * (C * kBlock);
    const char *src = a.src + a.src_rows.offset(row) * static_cast<int64_t>(sizeof(T));
    char *out = a.out + a.out_rows.offset(row) * static_cast<int64_t>(sizeof(T));
    u32x4 raw[C];
    bool inside[C];
#pragma unroll
    for (int c = 0; c < C; ++c) {
        const int64_t tile = first + c * kBlock + lane;
        inside[c] = tile < nvec;
        raw[c] = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(src + (inside[c] ? tile : nvec - 1) * 16));
    }
    __builtin_amdgcn_sched_barrier(0);
    // The row's maximum and sum from its slices': a lane folds slices lane, lane + 256, ... in that order, then
    // the lanes fold in a fixed tree.
    const SlicePartial *mine = a.partials + row * a.slices;
    double top = -__builtin_huge_val();
    for (int64_t j = lane; j < a.slices; j += kBlock) top = mine[j].max > top ? mine[j].max : top;
    top = row_fold<kBlock>(MaxOp{}, top, lds);
    double sum = 0.0;
    for (int64_t j = lane; j < a.slices; j += kBlock) {
        const SlicePartial part = mine[j];
        // A slice of -inf only has sum 0 and stays out (its scale would be exp(-inf - top), or NaN for a row of
        // -inf only, which comes out NaN below without it).
        if (part.sum != 0.0) sum += part.sum * rescale<X>(part.max - top);
    }
    sum = row_fold<kBlock>(SumOp{}, sum, lds);
    if (top == -__builtin_huge_val()) sum = __builtin_nan("");  // a row of -inf only: NaN, as exp(-inf - -inf) makes it
    const X mx = static_cast<X>(top);
    const E scale = LOG ? M::lg(sum) : M::scale(sum);
    const __amdgpu_buffer_rsrc_t out_row = __builtin_amdgcn_make_buffer_rsrc(out, 0, -1, 0x00020000);
#pragma unroll
    for (int c = 0; c < C; ++c) {
        const int64_t tile = first + c * kBlock + lane;
        X x[V];
        M::unpack(raw[c], x);
        decltype(M::logsoft(x[0], mx, scale)) res[V];
#pragma unroll
        for (int i = 0; i < V; ++i) {
            if constexpr (LOG) {
                res[i] = M::logsoft(x[i], mx, scale);
            } else if constexpr (M::kKeep) {
                res[i] = M::soft(x[i], mx, M::ex(x[i], mx), scale);
            } else {
                res[i] = M::soft(x[i], mx, E(0), scale);
            }
        }
        if (inside[c]) {
            // A row's bytes may pass 4 GiB: the buffer form (32-bit offsets) serves rows below that.
            if (a.stream_stores) __builtin_nontemporal_store(M::pack(res), reinterpret_cast<u32x4 *>(out + tile * 16));
            else __builtin_amdgcn_raw_buffer_store_b128(M::pack(res), out_row, static_cast<int>(tile * 16), 0, 17 /* sc0 sc1 */);
        }
    }
}

// ---- rows that run across memory: a softmax along an outer dimension ----------------------------------
//
// The rows' elements lie `si` apart and the rows themselves next to each other (softmax over dim 0 of a
// matrix, over the channels of [N, C, H, W]). A lane owns V adjacent rows - one 16-byte vector per position -
// and the workgroup's lanes split in 8 across (128 bytes of every position; 16 or 32 across were no faster) times
// RG row groups that take the positions in turn. Two passes over the source: the first keeps, per row, a running
// maximum and the sum of exponentials about it (when the maximum rises the sum is rescaled), folded across the
// row groups in a fixed order; the second writes. The second pass finds the tile in the memory-side cache when
// the tiles in flight fit it.
struct ColsArgs {
    char *out;
    const char *src;
    Walk out_outer, src_outer;  // the row dimensions outside the contiguous run
    int64_t inner;              // rows in the contiguous run
    int64_t tiles_per_run;      // tiles of kColsAcross * V rows in it
    int64_t n, so, si;
    int64_t tiles;
};

constexpr int kColsAcross = 8;

// (max, sum about it) of a row part; merging rescales the side with the lower maximum.
template <class X>
struct Running {
    X m;
    double s;
};
template <class X>
__device__ __forceinline__ Running<X> merge(Running<X> a, Running<X> b) {
    const X m = b.m > a.m ? b.m : a.m;
    // A side that holds nothing yet (sum 0: no element, or -inf only) stays out: its scale may be exp(-inf + inf).
    const double sa = a.s != 0.0 ? a.s * rescale<X>(static_cast<double>(a.m) - static_cast<double>(m)) : 0.0;
    const double sb = b.s != 0.0 ? b.s * rescale<X>(static_cast<double>(b.m) - static_cast<double>(m)) : 0.0;
    return Running<X>{m, sa + sb};
}

template <class T, int BLOCK, bool LOG>
__global__ void __launch_bounds__(BLOCK) softmax_cols_kernel(ColsArgs a) {
    using M = SoftmaxMath<T>;
    using X = typename M::X;
    using E = typename M::E;
    constexpr int V = 16 / static_cast<int>(sizeof(T));
    constexpr int RG = BLOCK / kColsAcross;   // row groups
    constexpr int kWaves = BLOCK / kWave;
    constexpr int kGroupsPerWave = kWave / kColsAcross;
    constexpr int U = 4;                      // positions in flight per lane
    __shared__ X lds_m[kWaves][kColsAcross * V];
    __shared__ double lds_s[kWaves][kColsAcross * V];
    const int across = threadIdx.x % kColsAcross, rg = threadIdx.x / kColsAcross;
    const X kLow = -__builtin_huge_valf();
    for (int64_t tile = blockIdx.x; tile < a.tiles; tile += gridDim.x) {
        const int64_t run = tile / a.tiles_per_run, in_run = tile - run * a.tiles_per_run;
        const int64_t row0 = (in_run * kColsAcross + across) * V;  // this lane's first row inside the run
        const bool live = row0 < a.inner;
        const int64_t r = live ? row0 : 0;
        const T *src = reinterpret_cast<const T *>(a.src) + a.src_outer.offset(run) + r;
        T *out = reinterpret_cast<T *>(a.out) + a.out_outer.offset(run) + r;
        // Pass 1.
        Running<X> state[V];
#pragma unroll
        for (int i = 0; i < V; ++i) state[i] = Running<X>{kLow, 0.0};
        for (int64_t k0 = rg; k0 < a.n; k0 += static_cast<int64_t>(U) * RG) {
            u32x4 raw[U];
            bool valid[U];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int64_t k = k0 + static_cast<int64_t>(u) * RG;
                valid[u] = k < a.n;
                raw[u] = *reinterpret_cast<const u32x4 *>(src + (valid[u] ? k : k0) * a.si);
            }
            X x[U][V];
#pragma unroll
            for (int u = 0; u < U; ++u) M::unpack(raw[u], x[u]);
            bool rose = false;
            X top[V];
#pragma unroll
            for (int i = 0; i < V; ++i) {
                X m = state[i].m;
#pragma unroll
                for (int u = 0; u < U; ++u) m = valid[u] && x[u][i] > m ? x[u][i] : m;
                top[i] = m;
                rose |= m != state[i].m && state[i].s != 0.0;
            }
            // Rescaling is rare after a row's first positions: the whole wave skips it when no lane needs it.
            if (__builtin_amdgcn_ballot_w64(rose) != 0) {
#pragma unroll
                for (int i = 0; i < V; ++i) {
                    if (state[i].s != 0.0) state[i].s *= rescale<X>(static_cast<double>(state[i].m) - static_cast<double>(top[i]));
                }
            }
#pragma unroll
            for (int i = 0; i < V; ++i) {
                state[i].m = top[i];
                // An element of -inf adds nothing, also while the running maximum is -inf (exp(-inf + inf) would
                // say NaN): the end of the pass sees a row that holds nothing else. A NaN adds itself.
                if constexpr (std::is_same_v<E, double>) {
                    double add = 0.0;
#pragma unroll
                    for (int u = 0; u < U; ++u) {
                        const double e = M::ex(x[u][i], top[i]);
                        add += valid[u] && x[u][i] != kLow ? e : 0.0;
                    }
                    state[i].s += add;
                } else {
                    // Halves: the batch's terms meet in f32, one f64 addition per batch; for log_softmax the
                    // terms that are exactly 1 are counted instead of added (see the registers kernel).
                    float e[U], ones = 0.0f;
#pragma unroll
                    for (int u = 0; u < U; ++u) {
                        e[u] = valid[u] && x[u][i] != kLow ? M::ex(x[u][i], top[i]) : 0.0f;
                        if constexpr (LOG) {
                            const bool one = e[u] == 1.0f;
                            ones += one ? 1.0f : 0.0f;
                            e[u] = one ? 0.0f : e[u];
                        }
                    }
                    static_assert(U == 4, "the pairwise sum below");
                    state[i].s += static_cast<double>((e[0] + e[1]) + (e[2] + e[3]));
                    if constexpr (LOG) state[i].s += static_cast<double>(ones);
                }
            }
        }
        // The row groups meet in two rounds, each by shuffles inside a wave (lanes 8, 16, 32 apart hold the same
        // rows) and through LDS across the waves, in a fixed order: first the rows' maxima; then every lane moves
        // its own sums to them - the only exponentials of the meeting, one per row and lane - and the sums add up.
        X mx[V];
#pragma unroll
        for (int i = 0; i < V; ++i) {
            X m = state[i].m;
#pragma unroll
            for (int step = kColsAcross; step < kWave; step <<= 1) {
                const X other = shfl_xor_any(m, step);
                m = other > m ? other : m;
            }
            mx[i] = m;
        }
        __syncthreads();  // the last tile's readers are done
        if ((threadIdx.x % kWave) < kColsAcross) {
#pragma unroll
            for (int i = 0; i < V; ++i) lds_m[threadIdx.x / kWave][across * V + i] = mx[i];
        }
        __syncthreads();
        double total[V];
#pragma unroll
        for (int i = 0; i < V; ++i) {
            X m = lds_m[0][across * V + i];
#pragma unroll
            for (int w = 1; w < kWaves; ++w) {
                const X other = lds_m[w][across * V + i];
                m = other > m ? other : m;
            }
            mx[i] = m;
            // Sums of nothing (no element yet, or -inf only) stay 0: their scale may be exp(-inf + inf).
            double s = state[i].s;
            if (s != 0.0 && state[i].m != m) s *= rescale<X>(static_cast<double>(state[i].m) - static_cast<double>(m));
#pragma unroll
            for (int step = kColsAcross; step < kWave; step <<= 1) s += shfl_xor_any(s, step);
            total[i] = s;
        }
        if ((threadIdx.x % kWave) < kColsAcross) {
#pragma unroll
            for (int i = 0; i < V; ++i) lds_s[threadIdx.x / kWave][across * V + i] = total[i];
        }
        __syncthreads();
        E scale[V];
#pragma unroll
        for (int i = 0; i < V; ++i) {
            double sum = lds_s[0][across * V + i];
#pragma unroll
            for (int w = 1; w < kWaves; ++w) sum += lds_s[w][across * V + i];
            if (mx[i] == kLow) sum = __builtin_nan("");  // a row of -inf only
            scale[i] = LOG ? M::lg(sum) : M::scale(sum);
        }
        (void)kGroupsPerWave;
        // Pass 2.
        for (int64_t k0 = rg; k0 < a.n; k0 += static_cast<int64_t>(U) * RG) {
            u32x4 raw[U];
            bool valid[U];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int64_t k = k0 + static_cast<int64_t>(u) * RG;
                valid[u] = k < a.n;
                raw[u] = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(src + (valid[u] ? k : k0) * a.si));
            }
#pragma unroll
            for (int u = 0; u < U; ++u) {
                X x[V];
                M::unpack(raw[u], x);
                decltype(M::logsoft(x[0], mx[0], scale[0])) res[V];
#pragma unroll
                for (int i = 0; i < V; ++i) {
                    if constexpr (LOG) res[i] = M::logsoft(x[i], mx[i], scale[i]);
                    else if constexpr (M::kKeep) res[i] = M::soft(x[i], mx[i], M::ex(x[i], mx[i]), scale[i]);
                    else res[i] = M::soft(x[i], mx[i], E(0), scale[i]);
                }
                const int64_t k = k0 + static_cast<int64_t>(u) * RG;
                if (valid[u] && live) __builtin_nontemporal_store(M::pack(res), reinterpret_cast<u32x4 *>(out + k * a.so));
            }
        }
    }
}

// The same rows when every lane's share of the positions fits its registers (C positions per lane, one 16-byte
// vector of V rows each): read once, all loads in flight together, written from the registers. The streaming
// form above pays the memory's latency once per batch of four positions and reads the source twice.
//
// Addresses are a lane's own offset plus a step per position that is the same
// for the whole workgroup (buffer instructions: the step travels in a scalar register), so a position in flight
// costs its four data registers and nothing else. The launch has checked that every offset fits 32 bits.
// A position past the row's end re-reads a valid one and is then set to -inf, which no phase notices: it never is
// a maximum and its exponential is an exact 0.

// Orders a value's whole computation before whatever volatile statement follows (the exponential's Horner steps
// are such statements): without it the compiler starts every exponential of a phase and finishes them late, each
// holding eight registers meanwhile.
template <class A>
__device__ __forceinline__ void settle(A &v) {
    asm volatile("" : "+v"(v));
}

template <class T>
__device__ __forceinline__ u32x4 lowest_pattern() {
    if constexpr (std::is_same_v<T, float>) return u32x4{0xFF800000u, 0xFF800000u, 0xFF800000u, 0xFF800000u};
    else if constexpr (std::is_same_v<T, double>) return u32x4{0u, 0xFFF00000u, 0u, 0xFFF00000u};
    else if constexpr (std::is_same_v<T, bf16_t>) return u32x4{0xFF80FF80u, 0xFF80FF80u, 0xFF80FF80u, 0xFF80FF80u};
    else return u32x4{0xFC00FC00u, 0xFC00FC00u, 0xFC00FC00u, 0xFC00FC00u};
}

template <class T, int BLOCK, int C, bool LOG>
// Four waves per SIMD (128 registers a lane), so that a compute unit holds workgroups in different phases.
__global__ void __launch_bounds__(BLOCK, 4) softmax_cols_regs_kernel(ColsArgs a) {
    using M = SoftmaxMath<T>;
    using X = typename M::X;
    using E = typename M::E;
    constexpr int V = 16 / static_cast<int>(sizeof(T));
    constexpr int kElem = static_cast<int>(sizeof(T));
    constexpr int ACROSS = kColsAcross;
    constexpr int RG = BLOCK / ACROSS;
    constexpr int kWaves = BLOCK / kWave;
    constexpr int kStream = 2;  // the nontemporal bit of a buffer instruction
    __shared__ X lds_m[kWaves][ACROSS * V];
    __shared__ double lds_s[kWaves][ACROSS * V];
    const int across = threadIdx.x % ACROSS, rg = threadIdx.x / ACROSS;
    const int wave = __builtin_amdgcn_readfirstlane(static_cast<int>(threadIdx.x) / kWave);
    const bool writer = (threadIdx.x % kWave) < ACROSS;
    const X kLow = -__builtin_huge_valf();
    const uint32_t step_in = static_cast<uint32_t>(RG * a.si * kElem), step_out = static_cast<uint32_t>(RG * a.so * kElem);
    const int part = static_cast<int>(a.n / RG);  // the first position group that is not whole
    for (int64_t tile = blockIdx.x; tile < a.tiles; tile += gridDim.x) {
        const int64_t run = tile / a.tiles_per_run, in_run = tile - run * a.tiles_per_run;
        const int64_t first = in_run * (ACROSS * V);  // the tile's first row inside the run
        const bool live = first + across * V < a.inner;
        const char *src = a.src + (a.src_outer.offset(run) + first) * kElem;
        char *out = a.out + (a.out_outer.offset(run) + first) * kElem;
        const __amdgpu_buffer_rsrc_t src_rs = __builtin_amdgcn_make_buffer_rsrc(const_cast<char *>(src), 0, -1, 0x00020000);
        const __amdgpu_buffer_rsrc_t out_rs = __builtin_amdgcn_make_buffer_rsrc(out, 0, -1, 0x00020000);
        const uint32_t lane_at = live ? static_cast<uint32_t>(across) * 16u : 0u;
        const uint32_t at_in = lane_at + static_cast<uint32_t>(rg) * static_cast<uint32_t>(a.si * kElem);
        const uint32_t at_out = lane_at + static_cast<uint32_t>(rg) * static_cast<uint32_t>(a.so * kElem);
        // The group that is cut short carries its whole offset in the lane's register, so that a lane past the
        // end can take position 0 instead; so do the groups after it.
        const uint32_t at_part = rg + static_cast<int64_t>(part) * RG < a.n ? at_in + static_cast<uint32_t>(part) * step_in : lane_at;
        u32x4 raw[C];
#pragma unroll
        for (int c = 0; c < C; ++c) {
            const bool whole = c < part;
            raw[c] = __builtin_amdgcn_raw_buffer_load_b128(src_rs, static_cast<int>(whole ? at_in : at_part),
                                                           static_cast<int>(whole ? c * step_in : 0u), kStream);
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int c = 0; c < C; ++c) {
            if (c >= part) {  // the same for the whole workgroup
                const bool valid = rg + static_cast<int64_t>(c) * RG < a.n;
                const u32x4 low = lowest_pattern<T>();
#pragma unroll
                for (int j = 0; j < 4; ++j) raw[c][j] = valid ? raw[c][j] : low[j];
            }
        }
        // The rows' maxima: this lane's positions, the wave's row groups (lanes ACROSS and more apart hold the
        // same rows), the waves through LDS.
        X mx[V];
#pragma unroll
        for (int i = 0; i < V; ++i) mx[i] = kLow;
        static_assert(C % 2 == 0, "positions are compared two at a time");
#pragma unroll
        for (int c = 0; c < C; c += 2) {
            X x[V], y[V];
            M::unpack(raw[c], x);
            M::unpack(raw[c + 1], y);
#pragma unroll
            for (int i = 0; i < V; ++i) {
                // NaNs stay out of the maximum, as in `x > mx ? x : mx` (the sums pick them up).
                mx[i] = max3(mx[i], x[i], y[i]);
            }
        }
#pragma unroll
        for (int i = 0; i < V; ++i) {
#pragma unroll
            for (int step = ACROSS; step < kWave; step <<= 1) {
                const X other = shfl_xor_any(mx[i], step);
                mx[i] = other > mx[i] ? other : mx[i];
            }
        }
        __syncthreads();  // the last tile's readers are done
        if (writer) {
#pragma unroll
            for (int i = 0; i < V; ++i) lds_m[wave][across * V + i] = mx[i];
        }
        __syncthreads();
#pragma unroll
        for (int i = 0; i < V; ++i) {
            X m = lds_m[0][across * V + i];
#pragma unroll
            for (int w = 1; w < kWaves; ++w) {
                const X other = lds_m[w][across * V + i];
                m = other > m ? other : m;
            }
            mx[i] = m;
        }
        // The sums about them, as the CPU forms them (exp(x - max), so a row of -inf only or one holding +inf or a
        // NaN comes out NaN by itself). Halves: a lane's terms meet in f32 (sixteen of them at most, against
        // results of 8 or 11 bits); for log_softmax the terms that are exactly 1 are counted instead of added (see
        // the rows kernel).
        using Part = std::conditional_t<std::is_same_v<E, double>, double, float>;
        Part sum[V], ones[LOG && !std::is_same_v<E, double> ? V : 1];
#pragma unroll
        for (int i = 0; i < V; ++i) sum[i] = 0;
        if constexpr (LOG && !std::is_same_v<E, double>) {
#pragma unroll
            for (int i = 0; i < V; ++i) ones[i] = 0;
        }
#pragma unroll
        for (int c = 0; c < C; ++c) {
            X x[V];
            forget(raw[c]);
            M::unpack(raw[c], x);
#pragma unroll
            for (int i = 0; i < V; ++i) {
                Part e = M::ex(x[i], mx[i]);
                if constexpr (LOG && !std::is_same_v<E, double>) {
                    const bool one = e == 1.0f;
                    ones[i] += one ? 1.0f : 0.0f;
                    e = one ? 0.0f : e;
                }
                sum[i] += e;
                settle(sum[i]);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
#pragma unroll
        for (int i = 0; i < V; ++i) {
            double s = static_cast<double>(sum[i]);
            if constexpr (LOG && !std::is_same_v<E, double>) s += static_cast<double>(ones[i]);
#pragma unroll
            for (int step = ACROSS; step < kWave; step <<= 1) s += shfl_xor_any(s, step);
            if (writer) lds_s[wave][across * V + i] = s;
        }
        __syncthreads();
        E scale[V];
#pragma unroll
        for (int i = 0; i < V; ++i) {
            double total = lds_s[0][across * V + i];
#pragma unroll
            for (int w = 1; w < kWaves; ++w) total += lds_s[w][across * V + i];
            scale[i] = LOG ? M::lg(total) : M::scale(total);
        }
#pragma unroll
        for (int c = 0; c < C; ++c) {
            X x[V];
            forget(raw[c]);
            M::unpack(raw[c], x);
            decltype(M::logsoft(x[0], mx[0], scale[0])) res[V];
#pragma unroll
            for (int i = 0; i < V; ++i) {
                if constexpr (LOG) res[i] = M::logsoft(x[i], mx[i], scale[i]);
                else if constexpr (M::kKeep) res[i] = M::soft(x[i], mx[i], M::ex(x[i], mx[i]), scale[i]);
                else res[i] = M::soft(x[i], mx[i], E(0), scale[i]);
                settle(res[i]);
            }
            if (rg + static_cast<int64_t>(c) * RG < a.n && live) {
                __builtin_amdgcn_raw_buffer_store_b128(M::pack(res), out_rs, static_cast<int>(at_out),
                                                       static_cast<int>(c * step_out), kStream);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    }
}

// ---- plan -----------------------------------------------------------------------------------------

struct SoftmaxPlan {
    bool regs = false;   // registers plan
    bool split = false;  // rows cut across workgroups (two launches, a workspace)
    bool cols = false;   // rows that run across memory, neighbours adjacent
    int group = kWave;   // lanes per row (registers, streaming), per slice (split) or per workgroup (cols)
    int tiles = 0;       // registers and split plans: 128-bit tiles per lane; cols: positions per lane, 0 streams
    int64_t slices = 0;  // split plan: slices of a row
};

// Chunks per lane of a slice of the split plan, and the smallest row it is worth cutting.
constexpr int slice_tiles(int elem) { return elem == 2 ? 16 : 8; }
constexpr int64_t kSplitRowBytes = int64_t{256} << 10;

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
    int64_t nrows = 1;
    for (int d = 0; d < ws.ndim; ++d) nrows *= ws.size[d];
    bool aligned = (n == 1 || si == 1) &&
                   reinterpret_cast<uintptr_t>(static_cast<char *>(src_rows.data) + src_rows.offset * elem) % 16 == 0;
    for (int d = 0; aligned && d < ws.ndim; ++d) aligned = (ws.stride[d] * elem) % 16 == 0;
    const int64_t tiles = (n + vec - 1) / vec;  // 128-bit tiles in a row
    if (aligned && n >= 16 && n % vec == 0) {
        // Lanes per row and chunks per lane, first fit. 16-bit rows stay packed (4 registers per chunk);
        // wider rows also keep their f64 exponentials (8 more registers per f32 chunk), so they spread over
        // two waves before a lane takes more than four chunks: more resident waves hide the row loads.
        // 16-bit rows past 16 384 elements go to 1024 lanes rather than to sixteen chunks on each of 256: a
        // [4096, 32000] bf16 softmax with inputs and results from HBM took 96-97 us that way and takes 90-91
        // with four chunks on each of 1024 lanes.
        struct Step {
            int group, tiles;
        };
        static const Step half_steps[] = {{kWave, 16}, {kBlock, 8}, {1024, 16}};
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
                break;
            }
        }
        // Cut the rows when they do not fit the registers of a workgroup, or when whole rows would leave most of
        // the GPU without work (fewer than 64 workgroups' worth) and a row is long enough to share.
        const int64_t per_slice = int64_t{slice_tiles(elem)} * kBlock;
        const int64_t slices = (tiles + per_slice - 1) / per_slice;
        const bool few = p.regs && nrows * p.group < 64 * kBlock && n * elem >= kSplitRowBytes;
        if ((!p.regs || few) && slices >= 2 && nrows * slices < (int64_t{1} << 31)) {
            p.regs = false;
            p.split = true;
            p.group = kBlock;
            p.tiles = slice_tiles(elem);
            p.slices = slices;
            return p;
        }
        if (p.regs) return p;
    }
    // Rows across memory with their neighbours adjacent: whole 16-byte vectors of V rows at every position.
    if (n >= 2 && si != 1 && ws.ndim >= 1 && ws.stride[0] == 1 && ws.size[0] % vec == 0 && (si * elem) % 16 == 0 &&
        reinterpret_cast<uintptr_t>(static_cast<char *>(src_rows.data) + src_rows.offset * elem) % 16 == 0) {
        bool outer = true;
        for (int d = 1; outer && d < ws.ndim; ++d) outer = (ws.stride[d] * elem) % 16 == 0;
        if (outer) {
            p.cols = true;
            // Lanes of a workgroup: 8 across times as many row groups as give a lane sixteen positions or fewer -
            // the rows are then read once, into registers; longer rows stream twice. (Narrower tiles, which
            // would fit longer rows, lose more than a second pass costs: 64- and 32-byte pieces of every
            // position took 1.8 and 4 times as long.)
            struct Form {
                int block, chunks;
            };
            static const Form forms[] = {{kBlock, 4}, {kBlock, 8}, {kBlock, 16}, {512, 16}};
            p.group = 512;
            p.tiles = 0;
            for (const Form &f : forms) {
                if (n <= int64_t{f.chunks} * (f.block / kColsAcross)) {
                    p.group = f.block;
                    p.tiles = f.chunks;
                    break;
                }
            }
            return p;
        }
    }
    p.regs = false;
    p.group = n <= 4096 ? kWave : kBlock;
    p.tiles = 0;
    return p;
}

template <class T, bool LOG>
void launch_split(const SoftmaxPlan &p, const SoftmaxArgs &a, void *workspace, hipStream_t stream) {
    SliceArgs s{};
    s.out = a.out;
    s.src = a.src;
    s.out_rows = a.out_rows;
    s.src_rows = a.src_rows;
    if (s.src_rows.ndim == 0) {  // one row
        s.src_rows.ndim = s.out_rows.ndim = 1;
        s.src_rows.size[0] = s.out_rows.size[0] = 1;
        s.src_rows.stride[0] = s.out_rows.stride[0] = 0;
    }
    s.nrows = a.nrows;
    s.n = a.n;
    s.slices = p.slices;
    s.partials = static_cast<SlicePartial *>(workspace);
    // Nontemporal stores for outputs far larger than the memory-side cache, and for rows whose bytes pass what
    // the buffer form of the store addresses.
    s.stream_stores = a.stream_stores || a.n * static_cast<int64_t>(sizeof(T)) >= kNarrowSpanBytes ? 1 : 0;
    constexpr int C = slice_tiles(static_cast<int>(sizeof(T)));
    const dim3 grid(static_cast<unsigned>(a.nrows * p.slices));
    // A source that the memory-side cache can hold is read through the caches the first time - when the first
    // launch is bound by its exponentials anyway (f32, f64: an [8, 4194304] f32 softmax 90 -> 86 us); the 16-bit
    // kernels wait for memory, and streaming loads serve them better both times (the same shape in bf16 45 -> 40 us).
    if (sizeof(T) >= 4 && a.nrows * a.n * static_cast<int64_t>(sizeof(T)) <= (int64_t{192} << 20)) {
        hipLaunchKernelGGL((softmax_slice_stats_kernel<T, C, LOG, true>), grid, dim3(kBlock), 0, stream, s);
    } else {
        hipLaunchKernelGGL((softmax_slice_stats_kernel<T, C, LOG, false>), grid, dim3(kBlock), 0, stream, s);
    }
    hipLaunchKernelGGL((softmax_slice_write_kernel<T, C, LOG>), grid, dim3(kBlock), 0, stream, s);
}

template <class T, bool LOG>
void launch_cols(const SoftmaxPlan &p, const SoftmaxArgs &a, hipStream_t stream) {
    constexpr int V = 16 / static_cast<int>(sizeof(T));
    constexpr int64_t kElem = static_cast<int64_t>(sizeof(T));
    ColsArgs c{};
    c.out = a.out;
    c.src = a.src;
    c.inner = a.src_rows.size[0];
    c.n = a.n;
    c.so = a.so;
    c.si = a.si;
    // The walks over the runs: the row dimensions past the first (one run: a single step of stride 0).
    c.src_outer.ndim = c.out_outer.ndim = a.src_rows.ndim > 1 ? a.src_rows.ndim - 1 : 1;
    c.src_outer.size[0] = c.out_outer.size[0] = 1;
    c.src_outer.stride[0] = c.out_outer.stride[0] = 0;
    for (int d = 1; d < a.src_rows.ndim; ++d) {
        c.src_outer.size[d - 1] = c.out_outer.size[d - 1] = a.src_rows.size[d];
        c.src_outer.stride[d - 1] = a.src_rows.stride[d];
        c.out_outer.stride[d - 1] = a.out_rows.stride[d];
    }
    const int64_t cap = 1 << 20;
    auto grid_for = [&](int across) {
        c.tiles_per_run = (c.inner + across * V - 1) / (across * V);
        c.tiles = c.tiles_per_run * (a.nrows / c.inner);
        return dim3(static_cast<unsigned>(c.tiles < cap ? c.tiles : cap));
    };
    int block = p.group, chunks = p.tiles;
    constexpr int across = kColsAcross;
    // The registers form addresses with 32-bit offsets from a tile's first element: every position a lane may
    // name, the ones past the row's end included, has to stay below 2^32.
    const int64_t pitch = (c.si > c.so ? c.si : c.so) * kElem;
    if (chunks != 0 && (pitch * chunks * (block / across) + 256 >= (int64_t{1} << 32) ||
                        static_cast<int64_t>(chunks) * (block / across) < c.n)) {
        chunks = 0;
        block = 512;
    }
    bool done = false;
    auto regs = [&](auto block_tag, auto chunks_tag) {
        constexpr int BLOCK = decltype(block_tag)::value, C = decltype(chunks_tag)::value;
        if (done || block != BLOCK || chunks != C) return;
        const dim3 grid = grid_for(kColsAcross);
        hipLaunchKernelGGL((softmax_cols_regs_kernel<T, BLOCK, C, LOG>), grid, dim3(BLOCK), 0, stream, c);
        done = true;
    };
    regs(IntTag<kBlock>{}, IntTag<4>{});
    regs(IntTag<kBlock>{}, IntTag<8>{});
    regs(IntTag<kBlock>{}, IntTag<16>{});
    regs(IntTag<512>{}, IntTag<16>{});
    if (done) return;
    // Streamed: two 512-lane workgroups a compute unit, so that one computes while the other waits for memory (a
    // [4096, 16384] f32 softmax along dim 0: 158 us, against 177 with one 1024-lane workgroup and 168 with four
    // of 256 lanes).
    (void)block;
    const dim3 grid = grid_for(kColsAcross);
    hipLaunchKernelGGL((softmax_cols_kernel<T, 512, LOG>), grid, dim3(512), 0, stream, c);
}

template <class T, bool LOG>
void launch_softmax(const SoftmaxPlan &p, const SoftmaxArgs &a, bool out_ok, bool out_cols, void *workspace, hipStream_t stream) {
    const int64_t cap = 1 << 20;
    if (p.split && out_ok) {
        launch_split<T, LOG>(p, a, workspace, stream);
        return;
    }
    if (p.cols && out_cols) {
        launch_cols<T, LOG>(p, a, stream);
        return;
    }
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
        const int group = p.group, tiles = p.tiles;
        auto with_tiles = [&](auto g) {
            switch (tiles) {
                case 1: run(g, IntTag<1>{}); break;
                case 2: run(g, IntTag<2>{}); break;
                case 4: run(g, IntTag<4>{}); break;
                case 8: run(g, IntTag<8>{}); break;
                default:
                    if constexpr (sizeof(T) == 2) run(g, IntTag<16>{});
                    break;
            }
        };
        if (group == kWave) with_tiles(IntTag<kWave>{});
        else if (group == 128) with_tiles(IntTag<128>{});
        else if (group == kBlock) with_tiles(IntTag<kBlock>{});
        else with_tiles(IntTag<1024>{});
        return;
    }
    const int group = p.regs || p.split || p.cols ? (a.n <= 4096 ? kWave : kBlock) : p.group;
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
        *bytes = 0;
        if (nrows == 0 || n == 0) return HMR_OK;
        hmr::Walk wo, ws;
        hmr::walk_pair(*src_rows, *src_rows, wo, ws);
        const hmr::SoftmaxPlan p = hmr::plan_softmax(*src_rows, n, src_stride, ws);
        // A split plan keeps a (maximum, sum) pair per slice of every row.
        if (p.split) *bytes = nrows * p.slices * static_cast<int64_t>(sizeof(hmr::SlicePartial));
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
        *split = p.split ? 1 : 0;
        *group = p.group;
        *cache = p.regs || p.split ? p.tiles * (16 / hmr::dtype_size(src_rows->dtype)) : 0;
        return HMR_OK;
    });
}

hmr_status hmr_softmax(hmr_context_t ctx, const hmr_tensor_desc *out_rows, const hmr_tensor_desc *src_rows, int64_t n,
                       int64_t out_stride, int64_t src_stride, int32_t log, void *workspace,
                       int64_t workspace_bytes) {
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
        // The output of a column plan: laid out like the source's rows (neighbours adjacent, everything aligned).
        bool out_cols = plan.cols && a.out_rows.ndim >= 1 && a.out_rows.stride[0] == 1 && (out_stride * elem) % 16 == 0 &&
                        reinterpret_cast<uintptr_t>(a.out) % 16 == 0;
        for (int d = 1; out_cols && d < a.out_rows.ndim; ++d) out_cols = (a.out_rows.stride[d] * elem) % 16 == 0;
        if (plan.split && out_ok) {
            const int64_t need = nrows * plan.slices * static_cast<int64_t>(sizeof(hmr::SlicePartial));
            if (workspace == nullptr || workspace_bytes < need) return hmr::fail(HMR_INVALID, "softmax: the workspace is too small");
        }
        return hmr::queue_on(ctx, "softmax", [&](hipStream_t stream) {
            if (out_rows->dtype != src_rows->dtype) return false;
            return hmr::with_float_type(out_rows->dtype, [&](auto t) {
                using T = typename decltype(t)::type;
                if (log != 0) hmr::launch_softmax<T, true>(plan, a, out_ok, out_cols, workspace, stream);
                else hmr::launch_softmax<T, false>(plan, a, out_ok, out_cols, workspace, stream);
            });
        });
    });
}

}  // extern "C"
