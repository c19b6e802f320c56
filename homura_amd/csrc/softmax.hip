// hmr_softmax / hmr_softmax_workspace / hmr_test_softmax_plan
// (ref: csrc/homura_rocm.h:338-346, csrc/reduce.hip:162-360, 519-584).
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
#include "reduce.hpp"

namespace hmr {
namespace {

// ---- exp in the evaluation type ------------------------------------------------------------------

// exp(t) for t <= 0 (or NaN) in f64. |relative error| < 2^-45.
__device__ __forceinline__ double exp_neg_f64(double t) {
    if (!(t >= -708.0)) return t != t ? t : 0.0;  // underflow region (and -inf) -> 0; NaN stays NaN
    const double kLog2e = 1.4426950408889634074;
    const double kLn2Hi = 6.93147180369123816490e-01;
    const double kLn2Lo = 1.90821492927058770002e-10;
    double n = rint(t * kLog2e);
    double r = fma(-n, kLn2Hi, t);
    r = fma(-n, kLn2Lo, r);  // |r| <= 0.3466
    // Taylor to degree 11: remainder < 0.3466^12 / 12! < 2^-47.
    double p = 1.0 / 39916800.0;
    p = fma(p, r, 1.0 / 3628800.0);
    p = fma(p, r, 1.0 / 362880.0);
    p = fma(p, r, 1.0 / 40320.0);
    p = fma(p, r, 1.0 / 5040.0);
    p = fma(p, r, 1.0 / 720.0);
    p = fma(p, r, 1.0 / 120.0);
    p = fma(p, r, 1.0 / 24.0);
    p = fma(p, r, 1.0 / 6.0);
    p = fma(p, r, 0.5);
    p = fma(p, r, 1.0);
    p = fma(p, r, 1.0);
    // Scale by 2^n, n in [-1022, 0]: add to the exponent field.
    int64_t bits = __double_as_longlong(p) + (static_cast<int64_t>(n) << 52);
    return __longlong_as_double(bits);
}

template <class T>
struct SoftmaxMath;

// Halves: values travel as f32.
template <class T>
struct HalfMath {
    using X = float;  // a row element in registers
    using E = float;  // exp(x - max), and the per-row scale
    static __device__ __forceinline__ X load(T v) { return Comp<T>::up(v); }
    static __device__ __forceinline__ E ex(X x, X mx) { return expf(x - mx); }
    static __device__ __forceinline__ double wide(E e) { return static_cast<double>(e); }
    static __device__ __forceinline__ E inv(double sum) { return static_cast<float>(sum); }  // keeps the sum; see soft()
    static __device__ __forceinline__ E lg(double sum) { return static_cast<float>(log(sum)); }
    static __device__ __forceinline__ T soft(E e, E sum) { return Comp<T>::down(e / sum); }
    static __device__ __forceinline__ T logsoft(X x, X mx, E log_sum) { return Comp<T>::down(x - mx - log_sum); }
};
template <>
struct SoftmaxMath<f16_t> : HalfMath<f16_t> {};
template <>
struct SoftmaxMath<bf16_t> : HalfMath<bf16_t> {};

template <>
struct SoftmaxMath<float> {
    using X = float;
    using E = double;
    static __device__ __forceinline__ X load(float v) { return v; }
    static __device__ __forceinline__ E ex(X x, X mx) { return exp_neg_f64(static_cast<double>(x) - static_cast<double>(mx)); }
    static __device__ __forceinline__ double wide(E e) { return e; }
    static __device__ __forceinline__ E inv(double sum) { return 1.0 / sum; }
    static __device__ __forceinline__ E lg(double sum) { return log(sum); }
    static __device__ __forceinline__ float soft(E e, E inv_sum) { return static_cast<float>(e * inv_sum); }
    static __device__ __forceinline__ float logsoft(X x, X mx, E log_sum) {
        return static_cast<float>(static_cast<double>(x) - static_cast<double>(mx) - log_sum);
    }
};

template <>
struct SoftmaxMath<double> {
    using X = double;
    using E = double;
    static __device__ __forceinline__ X load(double v) { return v; }
    static __device__ __forceinline__ E ex(X x, X mx) { return exp(x - mx); }
    static __device__ __forceinline__ double wide(E e) { return e; }
    static __device__ __forceinline__ E inv(double sum) { return sum; }
    static __device__ __forceinline__ E lg(double sum) { return log(sum); }
    static __device__ __forceinline__ double soft(E e, E sum) { return e / sum; }
    static __device__ __forceinline__ double logsoft(X x, X mx, E log_sum) { return x - mx - log_sum; }
};

// ---- combining across the lanes of a row ---------------------------------------------------------

struct MaxOp {
    using Acc = double;
    __device__ __forceinline__ Acc combine(Acc a, Acc b) const { return b > a ? b : a; }
};
struct MaxOpF {
    using Acc = float;
    __device__ __forceinline__ Acc combine(Acc a, Acc b) const { return b > a ? b : a; }
};
struct SumOp {
    using Acc = double;
    __device__ __forceinline__ Acc combine(Acc a, Acc b) const { return a + b; }
};

// Folds `v` over the G lanes that share a row (G = 64: one wave; else the whole workgroup).
template <int G, class Op>
__device__ __forceinline__ typename Op::Acc row_fold(const Op &op, typename Op::Acc v, typename Op::Acc *lds) {
    v = wave_fold(op, v);
    if constexpr (G > kWave) {
        constexpr int kWaves = G / kWave;
        __syncthreads();
        if (threadIdx.x % kWave == 0) lds[threadIdx.x / kWave] = v;
        __syncthreads();
        v = lds[0];
#pragma unroll
        for (int w = 1; w < kWaves; ++w) v = op.combine(v, lds[w]);
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
};

// Contiguous rows held in registers. G lanes per row, each with up to C tiles of V elements:
// tile c of lane l covers elements (c*G + l)*V .. +V, so every load of the group is one
// contiguous, coalesced span.
template <class T, int G, int C, bool LOG>
__global__ void __launch_bounds__(G > kBlock ? G : kBlock) softmax_regs_kernel(SoftmaxArgs a) {
    using M = SoftmaxMath<T>;
    using X = typename M::X;
    using E = typename M::E;
    using MaxFold = std::conditional_t<std::is_same_v<X, float>, MaxOpF, MaxOp>;
    constexpr int V = 16 / static_cast<int>(sizeof(T));
    constexpr int kThreads = G > kBlock ? G : kBlock;
    constexpr int kRowsPerBlock = kThreads / G;
    __shared__ double lds[G > kWave ? G / kWave : 1];
    const int lane = threadIdx.x % G;
    const int64_t groups = (a.nrows + kRowsPerBlock - 1) / kRowsPerBlock;
    const int64_t nvec = a.n / V;  // whole tiles in a row; the rest (< V elements) is the ragged end
    for (int64_t g = blockIdx.x; g < groups; g += gridDim.x) {
        const int64_t row = g * kRowsPerBlock + threadIdx.x / G;
        const bool live = row < a.nrows;
        const T *src = reinterpret_cast<const T *>(a.src) + (live ? a.src_rows.offset(row) : 0);
        T *out = reinterpret_cast<T *>(a.out) + (live ? a.out_rows.offset(row) : 0);
        X x[C][V];
        const X ninf = -__builtin_huge_valf();
        // Phase 0: one pass over memory.
#pragma unroll
        for (int c = 0; c < C; ++c) {
            const int64_t tile = static_cast<int64_t>(c) * G + lane;
            T raw[V];
            if (live && tile < nvec) {
                load_tile<T, V, kStreamLoads>(reinterpret_cast<const char *>(src + tile * V), raw);
#pragma unroll
                for (int i = 0; i < V; ++i) x[c][i] = M::load(raw[i]);
            } else {
#pragma unroll
                for (int i = 0; i < V; ++i) {
                    const int64_t e = tile * V + i;
                    // Past the row: -inf neither raises the max nor adds to the sum.
                    x[c][i] = (live && e < a.n) ? M::load(src[e]) : ninf;
                }
            }
        }
        // Phase 1: max. A NaN never replaces (v > m is false), as on the CPU.
        X mx = ninf;
#pragma unroll
        for (int c = 0; c < C; ++c) {
#pragma unroll
            for (int i = 0; i < V; ++i) mx = x[c][i] > mx ? x[c][i] : mx;
        }
        mx = row_fold<G>(MaxFold{}, mx, reinterpret_cast<X *>(lds));
        // Phase 2: exponentials and their f64 sum. Padding past the row must add exactly 0 even
        // when the row's max is -inf (where a real -inf entry yields NaN).
        double sum = 0.0;
        E ex[LOG ? 1 : C][LOG ? 1 : V];
#pragma unroll
        for (int c = 0; c < C; ++c) {
#pragma unroll
            for (int i = 0; i < V; ++i) {
                const int64_t e = (static_cast<int64_t>(c) * G + lane) * V + i;
                E v = M::ex(x[c][i], mx);
                if (!(e < a.n)) v = E(0);
                sum += M::wide(v);
                if constexpr (!LOG) ex[c][i] = v;
            }
        }
        sum = row_fold<G>(SumOp{}, sum, lds);
        // Phase 3: write once.
        const E scale = LOG ? M::lg(sum) : M::inv(sum);
#pragma unroll
        for (int c = 0; c < C; ++c) {
            const int64_t tile = static_cast<int64_t>(c) * G + lane;
            T res[V];
#pragma unroll
            for (int i = 0; i < V; ++i) {
                if constexpr (LOG) res[i] = M::logsoft(x[c][i], mx, scale);
                else res[i] = M::soft(ex[c][i], scale);
            }
            if (live && tile < nvec) {
                store_tile<T, V, kStreamStores>(reinterpret_cast<char *>(out + tile * V), res);
            } else if (live) {
#pragma unroll
                for (int i = 0; i < V; ++i) {
                    const int64_t e = tile * V + i;
                    if (e < a.n) out[e] = res[i];
                }
            }
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
    __shared__ double lds[G > kWave ? G / kWave : 1];
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
        const E scale = LOG ? M::lg(sum) : M::inv(sum);
        for (int64_t k = lane; k < n; k += G) {
            X v = M::load(src[k * a.si]);
            out[k * a.so] = LOG ? M::logsoft(v, mx, scale) : M::soft(M::ex(v, mx), scale);
        }
    }
}

// ---- plan -----------------------------------------------------------------------------------------

struct SoftmaxPlan {
    bool regs = false;  // registers plan (else streaming)
    int group = kWave;  // lanes per row
    int tiles = 0;      // registers plan: 128-bit tiles per lane
};

int64_t walk_pair(const hmr_tensor_desc &out_rows, const hmr_tensor_desc &src_rows, Walk &wo, Walk &ws) {
    // Merge the row dimensions with respect to both operands, innermost first.
    int64_t size[HMR_MAX_DIMS], so[HMR_MAX_DIMS], ss[HMR_MAX_DIMS];
    int n = 0;
    int64_t count = 1;
    for (int i = 0; i < src_rows.ndim; ++i) count *= src_rows.sizes[i];
    wo.ndim = ws.ndim = 0;
    if (count == 0) return 0;
    for (int i = 0; i < src_rows.ndim; ++i) {
        int64_t sz = src_rows.sizes[i];
        if (sz == 1) continue;
        int64_t p1 = 0, p2 = 0;
        if (n > 0 && !__builtin_mul_overflow(out_rows.strides[i], sz, &p1) && p1 == so[n - 1] &&
            !__builtin_mul_overflow(src_rows.strides[i], sz, &p2) && p2 == ss[n - 1]) {
            size[n - 1] *= sz;
            so[n - 1] = out_rows.strides[i];
            ss[n - 1] = src_rows.strides[i];
        } else {
            size[n] = sz;
            so[n] = out_rows.strides[i];
            ss[n] = src_rows.strides[i];
            ++n;
        }
    }
    wo.ndim = ws.ndim = n;
    for (int i = 0; i < n; ++i) {
        wo.size[i] = ws.size[i] = size[n - 1 - i];
        wo.stride[i] = so[n - 1 - i];
        ws.stride[i] = ss[n - 1 - i];
    }
    return count;
}

constexpr int kMaxTiles = 8;  // 128-bit tiles a lane keeps (8 x 16 B of the row)

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
    if (aligned && n >= 16) {
        for (int g : {kWave, kBlock, 1024}) {
            int64_t per = (tiles + g - 1) / g;
            if (per <= kMaxTiles) {
                p.regs = true;
                p.group = g;
                p.tiles = per <= 1 ? 1 : (per <= 2 ? 2 : (per <= 4 ? 4 : 8));
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
            hipLaunchKernelGGL((softmax_regs_kernel<T, G, C, LOG>), blocks(kThreads / G), dim3(kThreads), 0, stream, a);
        };
        auto with_tiles = [&](auto g) {
            switch (p.tiles) {
                case 1: run(g, IntTag<1>{}); break;
                case 2: run(g, IntTag<2>{}); break;
                case 4: run(g, IntTag<4>{}); break;
                default: run(g, IntTag<8>{}); break;
            }
        };
        if (p.group == kWave) with_tiles(IntTag<kWave>{});
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

hmr_status check_rows(const hmr_tensor_desc &out_rows, const hmr_tensor_desc &src_rows, int64_t n, int64_t so,
                      int64_t si, int64_t &nrows) {
    int64_t m = 0;
    if (hmr_status s = check_desc(out_rows, nrows)) return s;
    if (hmr_status s = check_desc(src_rows, m)) return s;
    bool same = out_rows.ndim == src_rows.ndim;
    for (int j = 0; same && j < out_rows.ndim; ++j) same = out_rows.sizes[j] == src_rows.sizes[j];
    if (!same) return fail(HMR_INVALID, "kernel operands have different sizes");
    if (n < 0 || so < 0 || si < 0) return fail(HMR_INVALID, "invalid softmax row");
    return HMR_OK;
}

}  // namespace
}  // namespace hmr

using hmr::guarded;

extern "C" {

hmr_status hmr_softmax_workspace(const hmr_tensor_desc *src_rows, int64_t n, int64_t src_stride, int64_t *bytes) {
    return guarded([&] {
        int64_t nrows = 0;
        if (hmr_status s = hmr::check_rows(*src_rows, *src_rows, n, 0, src_stride, nrows)) return s;
        *bytes = 0;  // no plan of this library cuts a row across workgroups
        return HMR_OK;
    });
}

hmr_status hmr_test_softmax_plan(const hmr_tensor_desc *src_rows, int64_t n, int64_t src_stride, int32_t *split,
                                 int32_t *group, int32_t *cache) {
    return guarded([&] {
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
    return guarded([&] {
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
        hmr::SoftmaxPlan plan = hmr::plan_softmax(*src_rows, n, src_stride, a.src_rows);
        bool out_ok = (n == 1 || out_stride == 1) && reinterpret_cast<uintptr_t>(a.out) % 16 == 0;
        for (int d = 0; out_ok && d < a.out_rows.ndim; ++d) out_ok = (a.out_rows.stride[d] * elem) % 16 == 0;
        return hmr::launch_on(ctx, "softmax", [&](hipStream_t stream) {
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
