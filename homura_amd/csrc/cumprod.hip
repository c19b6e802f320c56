// hmr_exclusive_cumprod (ref: csrc/homura_rocm.h:341-351, csrc/reduce.hip:397-417, 581-608; the semantics are
// src/backend/cpu/reduce.rs:227-324).
#include "dispatch.hpp"
#include "lines.hpp"
#include "reduce.hpp"

namespace hmr {
namespace {

// ---- the product of a line, one thread per line -------------------------------------------------------------
//
// out[k] = the product of the line's elements before k (after k when reversed), accumulated one
// element at a time in f32 (F16, BF16) or f64 (F32, F64) and rounded to the dtype as it is written;
// the accumulator is never rounded. Multiplication isn't associative, so a line is one thread's
// sequential loop, which is what fixes the bits: lines next to each other in memory are read
// coalesced across the threads, and a line that is itself contiguous is read and written in 16-byte
// tiles by its thread.
template <class T>
struct ProductOf {
    using A = float;
    static __device__ __forceinline__ A widen(T x) { return Comp<T>::up(x); }
    static __device__ __forceinline__ T narrow(A acc) { return Comp<T>::down(acc); }
};
template <>
struct ProductOf<float> {
    using A = double;
    static __device__ __forceinline__ A widen(float x) { return static_cast<double>(x); }
    static __device__ __forceinline__ float narrow(A acc) { return static_cast<float>(acc); }
};
template <>
struct ProductOf<double> {
    using A = double;
    static __device__ __forceinline__ A widen(double x) { return x; }
    static __device__ __forceinline__ double narrow(A acc) { return acc; }
};

struct CumprodArgs {
    char *out;
    const char *src;
    int64_t nlines, n, so, si;
    Walk out_lines, src_lines;
    int32_t reverse;
};

template <class T, int V>
__global__ void __launch_bounds__(kBlock) cumprod_kernel(CumprodArgs a) {
    using P = ProductOf<T>;
    for (int64_t line = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x; line < a.nlines;
         line += static_cast<int64_t>(gridDim.x) * kBlock) {
        const T *ps = reinterpret_cast<const T *>(a.src) + a.src_lines.offset(line);
        T *po = reinterpret_cast<T *>(a.out) + a.out_lines.offset(line);
        typename P::A acc = 1;
        // The chain of multiplications is sequential, the memory accesses need not be: kAhead elements (or
        // tiles: 128 bytes of the thread's own row) are loaded together, multiplied through in
        // order and written together.
        constexpr int kAhead = V == 1 ? 32 : 8;
        if constexpr (V == 1) {
            int64_t k = 0;
            for (; k + kAhead <= a.n; k += kAhead) {
                T x[kAhead];
#pragma unroll
                for (int j = 0; j < kAhead; ++j) x[j] = ps[(a.reverse ? a.n - 1 - (k + j) : k + j) * a.si];
#pragma unroll
                for (int j = 0; j < kAhead; ++j) {
                    po[(a.reverse ? a.n - 1 - (k + j) : k + j) * a.so] = P::narrow(acc);
                    acc = acc * P::widen(x[j]);
                }
            }
            for (; k < a.n; ++k) {
                const int64_t at = a.reverse ? a.n - 1 - k : k;
                const T x = ps[at * a.si];  // read before the write: the operands may be one buffer
                po[at * a.so] = P::narrow(acc);
                acc = acc * P::widen(x);
            }
        } else {
            const int64_t tiles = a.n / V;
            auto scan_tile = [&](T(&r)[V], T(&w)[V]) {
                if (a.reverse) {
#pragma unroll
                    for (int i = V - 1; i >= 0; --i) {
                        w[i] = P::narrow(acc);
                        acc = acc * P::widen(r[i]);
                    }
                } else {
#pragma unroll
                    for (int i = 0; i < V; ++i) {
                        w[i] = P::narrow(acc);
                        acc = acc * P::widen(r[i]);
                    }
                }
            };
            int64_t c = 0;
            for (; c + kAhead <= tiles; c += kAhead) {
                T r[kAhead][V], w[kAhead][V];
#pragma unroll
                for (int j = 0; j < kAhead; ++j) {
                    load_tile<T, V, false>(reinterpret_cast<const char *>(ps + (a.reverse ? tiles - 1 - (c + j) : c + j) * V), r[j]);
                }
#pragma unroll
                for (int j = 0; j < kAhead; ++j) scan_tile(r[j], w[j]);
#pragma unroll
                for (int j = 0; j < kAhead; ++j) {
                    store_tile<T, V, false>(reinterpret_cast<char *>(po + (a.reverse ? tiles - 1 - (c + j) : c + j) * V), w[j]);
                }
            }
            for (; c < tiles; ++c) {
                const int64_t at = (a.reverse ? tiles - 1 - c : c) * V;
                T r[V], w[V];
                load_tile<T, V, false>(reinterpret_cast<const char *>(ps + at), r);
                scan_tile(r, w);
                store_tile<T, V, false>(reinterpret_cast<char *>(po + at), w);
            }
        }
    }
}

// ---- slabs through LDS -----------------------------------------------------------------------------------------
//
// A thread per line ties the memory traffic to the lanes that own lines: 4096 columns are 64 waves, a handful of
// them per compute unit at best, each with a few hundred bytes in flight. Here a workgroup owns LN lines and walks
// them in slabs of 64 to 256 steps: ALL of its 256 lanes move a slab between memory and LDS with 16-byte accesses
// (the next two slabs' loads are in flight while this one is multiplied through), and the first LN lanes run the
// products - one sequential chain per line, in the CPU's order, out of LDS. ADJACENT: the lines lie next to each
// other in memory (a product along an outer dimension), so the 16-byte vectors run across lines and a slab is
// [step][line]; otherwise a line's steps are contiguous (a product along the innermost dimension), the vectors
// run along the line and a slab is [line][step].
constexpr int kSlabMovers = 256;                  // lanes that move slabs (four waves)
constexpr int kSlabBlock = kSlabMovers + kWave;   // and the wave that runs the chains
// Steps of a slab: 32 KB of elements, between 64 and 256 steps. Long slabs matter: a slab's chains run while the
// next slabs' loads are in flight, and a few dozen steps do not cover the memory's latency.
template <class T, int LN>
constexpr int slab_steps() {
    constexpr int fit = 32768 / (LN * static_cast<int>(sizeof(T)));
    return fit < 64 ? 64 : (fit > 256 ? 256 : fit);
}

struct SlabArgs {
    char *out;
    const char *src;
    Walk out_lines, src_lines;
    int64_t nlines, n, so, si;
    int32_t reverse;
};

// SHORT: slabs of 64 steps, a quarter of the LDS, so that two or three workgroups share a compute unit: for calls
// with more workgroups than compute units, where the neighbours' traffic covers a workgroup's waits.
template <class T, int LN, bool ADJACENT, bool SHORT>
__global__ void __launch_bounds__(kSlabBlock) cumprod_slab_kernel(SlabArgs a) {
    using P = ProductOf<T>;
    using A = typename P::A;
    constexpr int V = 16 / static_cast<int>(sizeof(T));
    constexpr int K = SHORT ? 64 : slab_steps<T, LN>();
    // LDS holds the slab as it lies in memory, in the tensor's own type, so that a 16-byte vector moves with one
    // LDS access: [step][line] when the lines are adjacent, else [line][step] with rows V elements longer than a
    // slab (an odd number of 16-byte slots apart: the chains' 16-byte accesses spread over the banks). The chains
    // convert as they go: for a lone wave an LDS instruction costs some 15 cycles whatever its width, a conversion
    // four to eight, so the fewer and wider LDS accesses win.
    constexpr int kPitch = ADJACENT ? LN : K + V;           // elements between LDS rows
    constexpr int kCells = (ADJACENT ? K : LN) * kPitch;
    constexpr int kVectors = LN * K / V;                    // 16-byte vectors of a slab
    constexpr int VPT = kVectors / kSlabMovers;             // per moving lane
    constexpr int kAcross = (ADJACENT ? LN : K) / V;        // vectors of one LDS row
    static_assert(VPT >= 1 && kVectors % kSlabMovers == 0 && kSlabMovers % kAcross == 0 && K % 16 == 0, "slab shape");
    // Two slabs each way: while the chains run through one, the movers fill the next and drain the one before.
    __shared__ __attribute__((aligned(16))) T in_slabs[2][kCells];
    __shared__ __attribute__((aligned(16))) T res_slabs[2][kCells];
    // Where step k of the slab's line l lies in LDS.
    auto cell = [](int l, int k) { return ADJACENT ? k * kPitch + l : l * kPitch + k; };
    const int64_t line0 = static_cast<int64_t>(blockIdx.x) * LN;
    const bool chains = threadIdx.x < kWave;                      // the first wave; the others move
    const int t = static_cast<int>(threadIdx.x);                  // a chain's line inside the workgroup's LN
    const int m = chains ? 0 : static_cast<int>(threadIdx.x) - kWave;  // a mover's number
    // Where this mover's vectors lie: in memory (element offsets without the slab's own) and in LDS.
    int64_t src_at[VPT], out_at[VPT];
    int line_of[VPT];  // the vector's (first) line inside the workgroup's LN
    bool mine[VPT];
    int step_of[VPT];  // ADJACENT: the vector's step inside the slab; else the first of its V steps
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
        const int v = m + i * kSlabMovers;
        const int row = v / kAcross, col = (v % kAcross) * V;
        const int64_t line = line0 + (ADJACENT ? col : row);
        mine[i] = line < a.nlines;
        const int64_t l = mine[i] ? line : 0;
        src_at[i] = a.src_lines.offset(l);
        out_at[i] = a.out_lines.offset(l);
        step_of[i] = ADJACENT ? row : col;
        line_of[i] = ADJACENT ? col : row;
    }
    const int64_t slabs = (a.n + K - 1) / K;
    // Slab s covers the steps [s K, s K + K) counted in the order of the product; reversed, those are the
    // positions n - 1 - step. `first` is the slab's lowest position, `rows` how many positions it has.
    auto bounds = [&](int64_t s, int64_t &first, int &rows) {
        const int64_t begin = s * K, end = begin + K < a.n ? begin + K : a.n;
        rows = static_cast<int>(end - begin);
        first = a.reverse ? a.n - end : begin;
    };
    // Two slabs are requested ahead of the one being multiplied through: with one, a workgroup has 32 KB in flight,
    // and 128 workgroups of them do not cover the memory's latency (a 537 MB pass took 348 us, 1.5 TB/s).
    u32x4 ahead[VPT], later[VPT];
    auto fetch = [&](int64_t s, u32x4(&into)[VPT]) {
        int64_t first;
        int rows;
        bounds(s, first, rows);
#pragma unroll
        for (int i = 0; i < VPT; ++i) {
            // Vectors past the slab's positions (the last slab of a line) read the slab's first position again.
            const bool inside = ADJACENT ? step_of[i] < rows : step_of[i] + V <= rows;
            const int64_t step = first + (inside ? step_of[i] : 0);
            const T *p = reinterpret_cast<const T *>(a.src) + src_at[i] + step * a.si;
            into[i] = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(p));
        }
    };
    // The chain of this lane's line over the slab's `count` positions. Sixteen steps at a time, and the next
    // sixteen elements are read while these are multiplied through: the chain's wave is alone on its SIMD, so
    // nothing else hides the LDS reads' latency. A batch is addressed from its lowest position, so that every
    // access is a base register plus a constant (pairs of steps, or whole 16-byte runs of them, in one access).
    A acc = 1;
    auto chain = [&](auto dir, const T *in, T *res, int count) {
        constexpr bool kForward = decltype(dir)::value > 0;
        constexpr int B = 16;
        const int batches = count / B;
        auto one = [&](int k) {
            const int at = cell(t, k);
            const T x = in[at];
            res[at] = P::narrow(acc);
            acc = acc * P::widen(x);
        };
        auto lowest = [&](int b) { return (kForward ? b : batches - 1 - b) * B; };  // the batch's lowest position
        auto load = [&](int b, T(&x)[B]) {
            const T *p = in + cell(t, lowest(b));
#pragma unroll
            for (int i = 0; i < B; ++i) x[i] = p[cell(0, i)];
        };
        auto run = [&](int b, const T(&x)[B]) {
            T *p = res + cell(t, lowest(b));
            T y[B];
#pragma unroll
            for (int ii = 0; ii < B; ++ii) {
                const int i = kForward ? ii : B - 1 - ii;
                y[i] = P::narrow(acc);
                acc = acc * P::widen(x[i]);
            }
#pragma unroll
            for (int i = 0; i < B; ++i) p[cell(0, i)] = y[i];
        };
        // Backwards, the positions past the last whole batch come first.
        if (!kForward) {
            for (int k = count - 1; k >= batches * B; --k) one(k);
        }
        if (batches > 0) {
            T x0[B], x1[B];
            load(0, x0);
            int b = 0;
            for (; b + 2 <= batches; b += 2) {
                // The barriers keep the scheduler from sinking a batch's reads down to its own multiplications.
                load(b + 1, x1);
                __builtin_amdgcn_sched_barrier(0);
                run(b, x0);
                __builtin_amdgcn_sched_barrier(0);
                load(b + 2 < batches ? b + 2 : b + 1, x0);
                __builtin_amdgcn_sched_barrier(0);
                run(b + 1, x1);
                __builtin_amdgcn_sched_barrier(0);
            }
            if (b < batches) run(b, x0);
        }
        if (kForward) {
            for (int k = batches * B; k < count; ++k) one(k);
        }
    };
    auto stage = [&](int buffer) {  // the slab in `ahead` into LDS; `later` moves up
#pragma unroll
        for (int i = 0; i < VPT; ++i) {
            *reinterpret_cast<u32x4 *>(&in_slabs[buffer][cell(line_of[i], step_of[i])]) = ahead[i];
        }
#pragma unroll
        for (int i = 0; i < VPT; ++i) ahead[i] = later[i];
    };
    auto drain = [&](int64_t s) {  // the results of slab s from LDS to memory
        int64_t first;
        int rows;
        bounds(s, first, rows);
#pragma unroll
        for (int i = 0; i < VPT; ++i) {
            const bool inside = ADJACENT ? step_of[i] < rows : step_of[i] + V <= rows;
            if (mine[i] && inside) {
                const u32x4 w = *reinterpret_cast<const u32x4 *>(&res_slabs[s & 1][cell(line_of[i], step_of[i])]);
                T *p = reinterpret_cast<T *>(a.out) + out_at[i] + (first + step_of[i]) * a.so;
                *reinterpret_cast<u32x4 *>(p) = w;
            }
        }
    };
    auto clamped = [&](int64_t s) { return s < slabs ? s : slabs - 1; };  // past the last slab: it again, unused
    if (!chains) {
        fetch(0, ahead);
        fetch(clamped(1), later);
        stage(0);
        fetch(clamped(2), later);
    }
    __syncthreads();
    // One barrier per slab. Between two of them the chains run through slab s while the movers write slab s - 1's
    // results to memory, put slab s + 1 into LDS and request slab s + 3: none of them touches a buffer the other
    // side uses in the same interval.
    for (int64_t s = 0; s < slabs; ++s) {
        if (chains) {
            if (t < LN && line0 + t < a.nlines) {
                int64_t first;
                int rows;
                bounds(s, first, rows);
                if (a.reverse) chain(IntTag<-1>{}, in_slabs[s & 1], res_slabs[s & 1], rows);
                else chain(IntTag<1>{}, in_slabs[s & 1], res_slabs[s & 1], rows);
            }
        } else {
            if (s > 0) drain(s - 1);
            if (s + 1 < slabs) {
                stage(static_cast<int>((s + 1) & 1));
                fetch(clamped(s + 3), later);
            }
        }
        __syncthreads();
    }
    if (!chains) drain(slabs - 1);
}

// Whether the slab kernel applies, and in which form (1: lines adjacent, 2: lines contiguous along their steps).
template <class T>
int slab_form(const CumprodArgs &a) {
    constexpr int V = 16 / static_cast<int>(sizeof(T));
    if (a.n < 128 || a.nlines < 16) return 0;
    if (reinterpret_cast<uintptr_t>(a.out) % 16 != 0 || reinterpret_cast<uintptr_t>(a.src) % 16 != 0) return 0;
    const int nd = a.src_lines.ndim;
    bool outer = true;  // every line starts on a 16-byte boundary
    for (int d = 1; d < nd; ++d) outer = outer && a.out_lines.stride[d] % V == 0 && a.src_lines.stride[d] % V == 0;
    if (!outer) return 0;
    if (nd >= 1 && a.out_lines.stride[0] == 1 && a.src_lines.stride[0] == 1 && a.src_lines.size[0] % V == 0 &&
        a.so % V == 0 && a.si % V == 0) {
        return 1;
    }
    if (a.so == 1 && a.si == 1 && a.n % V == 0 && (nd == 0 || (a.out_lines.stride[0] % V == 0 && a.src_lines.stride[0] % V == 0))) {
        return 2;
    }
    return 0;
}

template <class T>
void launch_cumprod(const CumprodArgs &a, hipStream_t stream) {
    constexpr int kVec = 16 / static_cast<int>(sizeof(T));
    if (const int form = slab_form<T>(a)) {
        SlabArgs s{a.out, a.src, a.out_lines, a.src_lines, a.nlines, a.n, a.so, a.si, a.reverse};
        if (s.src_lines.ndim == 0) {  // one line
            s.src_lines.ndim = s.out_lines.ndim = 1;
            s.src_lines.size[0] = s.out_lines.size[0] = 1;
            s.src_lines.stride[0] = s.out_lines.stride[0] = 0;
        }
        // 64 lines per workgroup; 32 when that leaves compute units without one and a slab's rows in memory stay
        // 128 bytes or more.
        const bool narrow = (a.nlines + 63) / 64 < 192 && (form == 2 || 32 * sizeof(T) >= 128);
        const int64_t lines = narrow ? 32 : 64;
        const dim3 grid(static_cast<unsigned>((a.nlines + lines - 1) / lines));
        if (grid.x < (1u << 30)) {
            auto run = [&](auto lines_tag, auto adjacent_tag) {
                constexpr int kLines = decltype(lines_tag)::value;
                constexpr bool kAdjacent = decltype(adjacent_tag)::value != 0;
                if (grid.x >= 512) hipLaunchKernelGGL((cumprod_slab_kernel<T, kLines, kAdjacent, true>), grid, dim3(kSlabBlock), 0, stream, s);
                else hipLaunchKernelGGL((cumprod_slab_kernel<T, kLines, kAdjacent, false>), grid, dim3(kSlabBlock), 0, stream, s);
            };
            if (form == 1 && narrow) run(IntTag<32>{}, IntTag<1>{});
            else if (form == 1) run(IntTag<64>{}, IntTag<1>{});
            else if (narrow) run(IntTag<32>{}, IntTag<0>{});
            else run(IntTag<64>{}, IntTag<0>{});
            return;
        }
    }
    bool tiles = a.so == 1 && a.si == 1 && a.n % kVec == 0 && reinterpret_cast<uintptr_t>(a.out) % 16 == 0 &&
                 reinterpret_cast<uintptr_t>(a.src) % 16 == 0;
    for (int d = 0; tiles && d < a.src_lines.ndim; ++d) {
        tiles = a.out_lines.stride[d] % kVec == 0 && a.src_lines.stride[d] % kVec == 0;
    }
    const int64_t want = (a.nlines + kBlock - 1) / kBlock;
    const unsigned grid = static_cast<unsigned>(want < (int64_t{1} << 22) ? want : (int64_t{1} << 22));
    if (tiles) hipLaunchKernelGGL((cumprod_kernel<T, kVec>), dim3(grid), dim3(kBlock), 0, stream, a);
    else hipLaunchKernelGGL((cumprod_kernel<T, 1>), dim3(grid), dim3(kBlock), 0, stream, a);
}

}  // namespace
}  // namespace hmr

using hmr::fenced;

extern "C" {

hmr_status hmr_exclusive_cumprod(hmr_context_t ctx, const hmr_tensor_desc *out_lines, const hmr_tensor_desc *src_lines,
                                 int64_t n, int64_t out_stride, int64_t src_stride, int32_t reverse) {
    return fenced([&] {
        int64_t nlines = 0;
        if (hmr_status s = hmr::check_rows(*out_lines, *src_lines, n, out_stride, src_stride, nlines)) return s;
        if (nlines == 0 || n == 0) return HMR_OK;
        hmr::CumprodArgs a{};
        const int elem = hmr::dtype_size(src_lines->dtype);
        a.out = static_cast<char *>(out_lines->data) + out_lines->offset * elem;
        a.src = static_cast<const char *>(src_lines->data) + src_lines->offset * elem;
        a.nlines = hmr::walk_pair(*out_lines, *src_lines, a.out_lines, a.src_lines);
        a.n = n;
        a.so = out_stride;
        a.si = src_stride;
        a.reverse = reverse != 0;
        return hmr::queue_on(ctx, "exclusive_cumprod", [&](hipStream_t stream) {
            if (out_lines->dtype != src_lines->dtype) return false;
            return hmr::with_float_type(out_lines->dtype, [&](auto t) {
                hmr::launch_cumprod<typename decltype(t)::type>(a, stream);
            });
        });
    });
}

}  // extern "C"
