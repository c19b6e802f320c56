// Reduction plans and the entry points hmr_reduce_workspace, hmr_reduce, hmr_var, hmr_arg_reduce,
// hmr_test_reduce_plan (ref: csrc/homura_rocm.h:297-336, csrc/reduce.hip:133-170, 432-517).
#include <algorithm>
#include <mutex>

#include "reduce_plan.hpp"

// Where hmr_reduce_static stages its partial results: a block inside the library's code object, so each
// GPU the library runs on holds its own copy at its own address until the process ends. In host code this
// name is only a handle for hipGetSymbolAddress (bind_reduce_scratch below); every use goes through the
// address that call returns, kept in the context.
static __device__ __align__(256) unsigned char scratch[HMR_REDUCE_STATIC_BYTES];

namespace hmr {
namespace {

// Merges a description's dimensions by its strides (size-1 dropped, contiguous neighbours joined)
// into a Walk, innermost first. Returns the element count (0 when a size is 0).
int64_t build_walk(const hmr_tensor_desc &d, Walk &w) {
    int64_t size[HMR_MAX_DIMS], stride[HMR_MAX_DIMS];
    int n = 0;
    int64_t count = 1;
    for (int i = 0; i < d.ndim; ++i) count *= d.sizes[i];
    w.ndim = 0;
    if (count == 0) return 0;
    for (int i = 0; i < d.ndim; ++i) {
        if (d.sizes[i] == 1) continue;
        int64_t prod = 0;
        if (n > 0 && !__builtin_mul_overflow(d.strides[i], d.sizes[i], &prod) && prod == stride[n - 1]) {
            size[n - 1] *= d.sizes[i];
            stride[n - 1] = d.strides[i];
        } else {
            size[n] = d.sizes[i];
            stride[n] = d.strides[i];
            ++n;
        }
    }
    w.ndim = n;
    for (int i = 0; i < n; ++i) {
        w.size[i] = size[n - 1 - i];
        w.stride[i] = stride[n - 1 - i];
    }
    return count;
}

int64_t ceil_div(int64_t a, int64_t b) { return a / b + (a % b != 0); }

// Cuts nred into at most `want` slices of a multiple of `quantum` elements.
void cut(ReducePlan &p, int64_t want, int64_t quantum) {
    int64_t nred = p.args.nred;
    if (want <= 1 || nred <= quantum) {
        p.splits = 1;
        p.chunk = nred;
        return;
    }
    int64_t chunk = ceil_div(ceil_div(nred, want), quantum) * quantum;
    p.chunk = chunk;
    p.splits = ceil_div(nred, chunk);
    if (p.splits <= 1) {
        p.splits = 1;
        p.chunk = nred;
    }
}

}  // namespace

hmr_status plan_reduction(const hmr_tensor_desc *out, const hmr_tensor_desc &kept, const hmr_tensor_desc &red,
                          ReducePlan &p) {
    int64_t n = 0;
    if (hmr_status s = check_desc(kept, n)) return s;
    if (hmr_status s = check_desc(red, n)) return s;
    if (red.dtype != kept.dtype) return fail(HMR_INVALID, "reduction descriptions differ");
    if (out != nullptr) {
        if (hmr_status s = check_desc(*out, n)) return s;
        bool same = out->ndim == kept.ndim;
        int64_t stride = 1;
        for (int k = kept.ndim - 1; same && k >= 0; --k) {
            same = out->sizes[k] == kept.sizes[k] && (out->sizes[k] == 1 || out->strides[k] == stride);
            stride *= kept.sizes[k];
        }
        if (!same) return fail(HMR_INVALID, "a reduction's output is not contiguous with its sizes");
    }
    const int elem = dtype_size(kept.dtype);
    ReduceArgs &a = p.args;
    a.src = static_cast<const char *>(kept.data) + kept.offset * elem;
    a.nout = build_walk(kept, a.kept);
    a.nred = build_walk(red, a.red);
    a.partials = nullptr;
    a.runs = Runs{};
    p.kind = ReduceKind::Any;
    p.group = 1;
    p.splits = 1;
    p.chunk = a.nred;
    p.rstride = 0;
    p.inner = 0;
    p.across = 4;
    if (a.nout == 0 || a.nred == 0) return HMR_OK;  // nothing to read: one lane per output writes the identity

    const bool base_aligned = reinterpret_cast<uintptr_t>(a.src) % 16 == 0;
    auto strides_aligned = [&](const Walk &w, int from) {
        for (int d = from; d < w.ndim; ++d) {
            if ((w.stride[d] * elem) % 16 != 0) return false;
        }
        return true;
    };
    const bool red_contiguous = a.red.ndim == 1 && a.red.stride[0] == 1;
    const int vec = 16 / elem;
    // Rows: one contiguous run per output.
    if (red_contiguous && a.nred >= 256 && base_aligned && strides_aligned(a.kept, 0)) {
        p.kind = ReduceKind::Rows;
        if (a.nout * kWave >= kTargetLanes / 2 || a.nred <= 2048) {
            p.group = kWave;
        } else {
            p.group = kBlock;
            if (a.nout * kBlock < kTargetLanes / 2) cut(p, ceil_div(2 * kTargetLanes, a.nout * kBlock), 4096);
        }
        return HMR_OK;
    }
    // Rows over several runs: one reduced dimension has stride 1 and holds whole aligned vectors, up to three
    // others count the runs (whatever their order: a folded range may be walked in any order, and max/min are
    // told each element's position in the CPU's order).
    if (a.red.ndim >= 2 && a.red.ndim <= kRunDims + 1 && base_aligned && strides_aligned(a.kept, 0) &&
        a.nred / vec < (int64_t{1} << 31)) {
        int inner = -1;
        for (int d = 0; d < a.red.ndim && inner < 0; ++d) {
            if (a.red.stride[d] == 1 && a.red.size[d] % vec == 0 && a.red.size[d] * elem >= 256) inner = d;
        }
        bool ok = inner >= 0;
        for (int d = 0; ok && d < a.red.ndim; ++d) ok = d == inner || (a.red.stride[d] * elem) % 16 == 0;
        if (ok) {
            Runs &r = a.runs;
            int64_t pos = 1;
            r.dims = 0;
            for (int d = 0; d < a.red.ndim; ++d) {
                if (d == inner) {
                    r.length = static_cast<uint32_t>(a.red.size[d]);
                    r.vectors = make_fastdiv(static_cast<uint32_t>(a.red.size[d] / vec));
                    r.inner_pos = pos;
                } else {
                    r.size[r.dims] = make_fastdiv(static_cast<uint32_t>(a.red.size[d]));
                    r.stride[r.dims] = a.red.stride[d];
                    r.pos[r.dims] = pos;
                    ++r.dims;
                }
                pos *= a.red.size[d];
            }
            p.kind = ReduceKind::Rows;
            if (a.nout * kWave >= kTargetLanes / 2 || a.nred <= 2048) {
                p.group = kWave;
            } else {
                p.group = kBlock;
                if (a.nout * kBlock < kTargetLanes / 2) cut(p, ceil_div(2 * kTargetLanes, a.nout * kBlock), 4096);
            }
            return HMR_OK;
        }
    }
    // Cols: a contiguous run of outputs, one strided reduced dimension (fewer than 2^31 - 2^16 rows: the kernel
    // counts rows in 32 bits, and steps past the last one by the rows of all its slices' row groups at most).
    if (a.red.ndim == 1 && a.nred < (int64_t{1} << 31) - (int64_t{1} << 16) && a.kept.ndim >= 1 && a.kept.stride[0] == 1 &&
        a.kept.size[0] >= 32 && base_aligned && (a.red.stride[0] * elem) % 16 == 0 && strides_aligned(a.kept, 1)) {
        p.kind = ReduceKind::Cols;
        p.rstride = a.red.stride[0];
        p.inner = a.kept.size[0];
        // The kernel walks the outer kept dimensions only.
        for (int d = 1; d < a.kept.ndim; ++d) {
            a.kept.size[d - 1] = a.kept.size[d];
            a.kept.stride[d - 1] = a.kept.stride[d];
        }
        a.kept.ndim -= 1;
        // As many waves side by side as the run of outputs fills (wide spans read best).
        p.across = p.inner > 2 * kWave * vec ? 4 : (p.inner > kWave * vec ? 2 : 1);
        const int64_t tiles = ceil_div(p.inner, int64_t{p.across} * kWave * vec) * (a.nout / p.inner);
        // 1024-lane workgroups (16 / across row groups that meet in LDS: a sixteenth of the partial results
        // of single waves) where the columns are long enough to feed them and the tile's states fit LDS
        // (elements of four bytes or more).
        const bool big = a.nred >= 512 && elem >= 4;
        p.group = (big ? 1024 : kBlock) / kWave;
        const int64_t rgroups = p.group / p.across;
        // How many workgroups stream at once decides the rate, and more is not better: on 16384 x 4096 f32
        // (4 tiles) 32 slices run at 46 us, 44 to 48 at 39 us, 56 at 40.6, 64 (a workgroup on every compute
        // unit) at 40.4-41.8, 96 at 47. The plan aims at 184 workgroups of 1024 lanes (the same number of
        // waves with 256-lane workgroups), and keeps a slice long enough that its partial results stay
        // small beside the rows it read.
        const int64_t target = big ? 184 : 736;
        const int64_t min_rows = std::max<int64_t>(8 * rgroups, 256 / elem);
        int64_t want = (target + tiles / 2) / tiles;
        want = std::min(want, a.nred / min_rows);
        p.splits = want > 1 ? want : 1;
        p.chunk = ceil_div(a.nred, p.splits);  // rows per slice (they are interleaved, not consecutive)
        return HMR_OK;
    }
    // Any layout.
    p.group = a.nred <= 32 ? 1 : (a.nred <= 4096 ? kWave : kBlock);
    if (a.nout * p.group < kTargetLanes / 2 && a.nred > 4096) {
        cut(p, ceil_div(kTargetLanes, a.nout * p.group), 1024);
    }
    return HMR_OK;
}

int64_t means_bytes(const ReducePlan &p, bool var) {
    if (!var || p.args.nout == 0) return 0;
    return (p.args.nout * 8 + 255) / 256 * 256;
}

int64_t partial_bytes(const ReducePlan &p, bool var) {
    return p.splits > 1 ? p.splits * p.args.nout * (var ? kVarPartialBytes : kPartialBytes) : 0;
}

namespace {

// Checks the workspace and returns where the partials start.
hmr_status take_workspace(const ReducePlan &p, bool var, void *workspace, int64_t bytes, void *&partials) {
    int64_t need = means_bytes(p, var) + partial_bytes(p, var);
    if (need > 0 && (workspace == nullptr || bytes < need)) {
        return fail(HMR_INVALID, "a reduction's workspace is too small");
    }
    partials = need > 0 ? static_cast<char *>(workspace) + means_bytes(p, var) : nullptr;
    return HMR_OK;
}

void *element0(const hmr_tensor_desc &d) { return static_cast<char *>(d.data) + d.offset * dtype_size(d.dtype); }

bool is_float(int d) { return d >= HMR_F16 && d <= HMR_F64; }

// One reduction, planned and queued; the body of hmr_reduce and hmr_reduce_static.
hmr_status run_reduce(hmr_context_t ctx, int32_t op, const hmr_tensor_desc *out, const hmr_tensor_desc *kept,
                      const ReducePlan &p, void *partials) {
    if (p.args.nout == 0) return HMR_OK;
    if ((op == HMR_REDUCE_MAX || op == HMR_REDUCE_MIN) && p.args.nred == 0) {
        return fail(HMR_INVALID, "reduction over an empty dimension");
    }
    return queue_on(ctx, "reduce", [&](hipStream_t stream) {
        const int dtype = kept->dtype;
        void *o = element0(*out);
        switch (op) {
            case HMR_REDUCE_SUM:
            case HMR_REDUCE_PROD:
            case HMR_REDUCE_MEAN:
                if (is_float(dtype)) {
                    if (out->dtype != dtype) return false;
                    return launch_float_reduce(op, dtype, p, partials, o, stream);
                }
                if (op == HMR_REDUCE_MEAN || out->dtype != HMR_I64) return false;
                return launch_int_reduce(op, dtype, p, partials, o, stream);
            case HMR_REDUCE_MAX:
            case HMR_REDUCE_MIN:
                if (out->dtype != dtype) return false;
                return launch_extreme_reduce(op == HMR_REDUCE_MAX, dtype, p, partials, o, nullptr, stream);
            case HMR_REDUCE_ALL:
            case HMR_REDUCE_ANY:
                if (out->dtype != (dtype == HMR_U8 ? HMR_U8 : HMR_BOOL)) return false;
                return launch_truth_reduce(op, dtype, p, partials, o, stream);
            default: return false;
        }
    });
}

}  // namespace

namespace {
// The block belongs to one context per GPU at a time: the first one that stages partial results in it, until
// that context is destroyed. Two contexts have two streams, and their kernels would overwrite each other's
// partial results.
std::mutex owners_lock;
constexpr int kMaxDevices = 64;
const hmr_context *owners[kMaxDevices];

hmr_status claim_reduce_scratch(const hmr_context *ctx) {
    if (ctx->device < 0 || ctx->device >= kMaxDevices) return fail(HMR_INVALID, "hmr_reduce_static: device out of range");
    std::lock_guard<std::mutex> lock(owners_lock);
    if (owners[ctx->device] == nullptr) owners[ctx->device] = ctx;
    if (owners[ctx->device] == ctx) return HMR_OK;
    return fail(HMR_INVALID, "hmr_reduce_static: the static block of rocm:" + std::to_string(ctx->device) +
                                 " is in use by another context; call hmr_reduce with a workspace");
}
}  // namespace

void release_reduce_scratch(const hmr_context &ctx) noexcept {
    if (ctx.device < 0 || ctx.device >= kMaxDevices) return;
    std::lock_guard<std::mutex> lock(owners_lock);
    if (owners[ctx.device] == &ctx) owners[ctx.device] = nullptr;
}

hmr_status bind_reduce_scratch(hmr_context &ctx) {
    void *address = nullptr;
    const hipError_t found = hipGetSymbolAddress(&address, HIP_SYMBOL(::scratch));
    if (found != hipSuccess) return hip_failure(found, "hipGetSymbolAddress(&address, HIP_SYMBOL(scratch))");
    if (address == nullptr) return fail(HMR_INTERNAL_ERROR, "the static reduction block has no device address");
    ctx.reduce_scratch = address;
    return HMR_OK;
}

}  // namespace hmr

using hmr::fenced;

extern "C" {

hmr_status hmr_reduce_workspace(const hmr_tensor_desc *kept, const hmr_tensor_desc *red, int32_t var,
                                int64_t *bytes) {
    return fenced([&] {
        hmr::ReducePlan p;
        if (hmr_status s = hmr::plan_reduction(nullptr, *kept, *red, p)) return s;
        *bytes = hmr::means_bytes(p, var != 0) + hmr::partial_bytes(p, var != 0);
        return HMR_OK;
    });
}

hmr_status hmr_test_reduce_plan(const hmr_tensor_desc *kept, const hmr_tensor_desc *red, int64_t *group,
                                int64_t *splits, int64_t *chunk) {
    return fenced([&] {
        hmr::ReducePlan p;
        if (hmr_status s = hmr::plan_reduction(nullptr, *kept, *red, p)) return s;
        *group = p.group;
        *splits = p.splits;
        *chunk = p.chunk;
        return HMR_OK;
    });
}

hmr_status hmr_reduce(hmr_context_t ctx, int32_t op, const hmr_tensor_desc *out, const hmr_tensor_desc *kept,
                      const hmr_tensor_desc *red, void *workspace, int64_t workspace_bytes) {
    return fenced([&] {
        hmr::ReducePlan p;
        if (hmr_status s = hmr::plan_reduction(out, *kept, *red, p)) return s;
        void *partials = nullptr;
        if (hmr_status s = hmr::take_workspace(p, false, workspace, workspace_bytes, partials)) return s;
        return hmr::run_reduce(ctx, op, out, kept, p, partials);
    });
}

hmr_status hmr_reduce_static(hmr_context_t ctx, int32_t op, const hmr_tensor_desc *out, const hmr_tensor_desc *kept,
                             const hmr_tensor_desc *red) {
    return fenced([&] {
        if (ctx == nullptr) return hmr::fail(HMR_INVALID, "hmr_reduce_static: null context");
        hmr::ReducePlan p;
        if (hmr_status s = hmr::plan_reduction(out, *kept, *red, p)) return s;
        const int64_t need = hmr::partial_bytes(p, false);
        if (need > HMR_REDUCE_STATIC_BYTES) {
            return hmr::fail(HMR_INVALID, "hmr_reduce_static: this reduction stages " + std::to_string(need) +
                                              " bytes of partial results, the library's block holds " +
                                              std::to_string(HMR_REDUCE_STATIC_BYTES) +
                                              "; call hmr_reduce with a workspace");
        }
        if (need > 0) {
            if (hmr_status s = hmr::claim_reduce_scratch(ctx)) return s;
        }
        // Every partial result the second kernel reads is written by the first one of the same call, so
        // what an earlier call left in the block needs no clearing.
        return hmr::run_reduce(ctx, op, out, kept, p, need > 0 ? ctx->reduce_scratch : nullptr);
    });
}

hmr_status hmr_var(hmr_context_t ctx, const hmr_tensor_desc *out, const hmr_tensor_desc *kept,
                   const hmr_tensor_desc *red, double correction, int32_t take_sqrt, void *workspace,
                   int64_t workspace_bytes) {
    return fenced([&] {
        hmr::ReducePlan p;
        if (hmr_status s = hmr::plan_reduction(out, *kept, *red, p)) return s;
        void *partials = nullptr;
        if (hmr_status s = hmr::take_workspace(p, true, workspace, workspace_bytes, partials)) return s;
        if (p.args.nout == 0) return HMR_OK;
        return hmr::queue_on(ctx, "var", [&](hipStream_t stream) {
            if (out->dtype != kept->dtype || !hmr::is_float(kept->dtype)) return false;
            double *means = static_cast<double *>(workspace);
            double divisor = static_cast<double>(p.args.nred) - correction;
            divisor = divisor > 0.0 ? divisor : 0.0;
            if (hmr::launch_var_single_pass(kept->dtype, p, partials, hmr::element0(*out), divisor, take_sqrt != 0,
                                            stream)) {
                return true;
            }
            if (!hmr::launch_mean_pass(kept->dtype, p, partials, means, stream)) return false;
            return hmr::launch_deviation_pass(kept->dtype, p, partials, means, hmr::element0(*out), divisor,
                                              take_sqrt != 0, stream);
        });
    });
}

hmr_status hmr_arg_reduce(hmr_context_t ctx, const hmr_tensor_desc *values, const hmr_tensor_desc *indices,
                          const hmr_tensor_desc *kept, const hmr_tensor_desc *red, int32_t is_max, void *workspace,
                          int64_t workspace_bytes) {
    return fenced([&] {
        hmr::ReducePlan p;
        if (hmr_status s = hmr::plan_reduction(indices, *kept, *red, p)) return s;
        if (values != nullptr) {
            hmr::ReducePlan q;
            if (hmr_status s = hmr::plan_reduction(values, *kept, *red, q)) return s;
        }
        void *partials = nullptr;
        if (hmr_status s = hmr::take_workspace(p, false, workspace, workspace_bytes, partials)) return s;
        if (p.args.nred == 0) return hmr::fail(HMR_INVALID, "arg reduction of an empty dimension");
        if (p.args.nout == 0) return HMR_OK;
        return hmr::queue_on(ctx, "arg_reduce", [&](hipStream_t stream) {
            if (indices->dtype != HMR_I64) return false;
            if (values != nullptr && values->dtype != kept->dtype) return false;
            return hmr::launch_extreme_reduce(is_max != 0, kept->dtype, p, partials,
                                              values ? hmr::element0(*values) : nullptr, hmr::element0(*indices),
                                              stream);
        });
    });
}

}  // extern "C"
