// hmr_unary (ref: csrc/homura_rocm.h:202, csrc/elementwise.hip:996-1007).
#include "ew_common.hpp"
#include "map_table.hpp"

namespace hmr {
namespace {

// 16-bit operations that go through a result table when the tensor is large: everything that costs
// more than a handful of instructions per element.
constexpr int kFirstTableOp = HMR_UNARY_EXP, kLastTableOp = HMR_UNARY_GELU_TANH;
constexpr int kTableOps = kLastTableOp - kFirstTableOp + 1;
constexpr int kTableSlots = 2 * kTableOps;  // f16, bf16

int table_slot(int op, int dtype) { return (dtype == HMR_BF16 ? kTableOps : 0) + (op - kFirstTableOp); }

using FloatOps = std::integer_sequence<int, HMR_UNARY_NEG, HMR_UNARY_ABS, HMR_UNARY_SIGN, HMR_UNARY_RELU,
                                       HMR_UNARY_EXP, HMR_UNARY_LOG, HMR_UNARY_SQRT, HMR_UNARY_RSQRT,
                                       HMR_UNARY_RECIPROCAL, HMR_UNARY_SIN, HMR_UNARY_COS, HMR_UNARY_ERF,
                                       HMR_UNARY_TANH, HMR_UNARY_SIGMOID, HMR_UNARY_LOG_SIGMOID, HMR_UNARY_SILU,
                                       HMR_UNARY_GELU, HMR_UNARY_GELU_TANH>;
using IntOps = std::integer_sequence<int, HMR_UNARY_NEG, HMR_UNARY_ABS, HMR_UNARY_SIGN, HMR_UNARY_RELU>;

bool pick_unary(hmr_context_t ctx, int op, int out_dtype, int dtype, const MapCall &call, hipStream_t stream) {
    if (op == HMR_UNARY_LOGICAL_NOT) {
        if (out_dtype != HMR_BOOL) return false;
        return with_any_type(dtype, [&](auto t) {
            using T = typename decltype(t)::type;
            launch_map<LogicalNot<T>>(call, stream);
        });
    }
    if (out_dtype != dtype) return false;
    if (dtype == HMR_BOOL) {
        if (op != HMR_UNARY_SIGN) return false;  // the CPU has no other bool arm
        launch_map<Move<uint8_t>>(call, stream);
        return true;
    }
    bool done = false;
    if (with_int_type(dtype, [&](auto t) {
            using T = typename decltype(t)::type;
            done = with_code(op, IntOps{}, [&](auto o) { launch_map<UnaryInt<decltype(o)::value, T>>(call, stream); });
        })) {
        return done;
    }
    with_float_type(dtype, [&](auto t) {
        using T = typename decltype(t)::type;
        done = with_code(op, FloatOps{}, [&](auto o) {
            using F = UnaryFloat<decltype(o)::value, T>;
            if constexpr (sizeof(T) == 2 && decltype(o)::value >= kFirstTableOp && decltype(o)::value <= kLastTableOp) {
                if (ctx->tables != nullptr && table_applies<F>(call)) {
                    const int slot = table_slot(op, dtype);
                    launch_table<F>(call, reinterpret_cast<uint16_t *>(static_cast<char *>(ctx->tables) + slot * kTableBytes), stream);
                    return;
                }
            }
            launch_map<F>(call, stream);
        });
    });
    return done;
}

}  // namespace

// Every table of the context, allocated and filled before hmr_context_create returns, so that hmr_unary never
// allocates and never queues anything but the operation itself (a caller may be capturing the stream into a
// graph, where a fill would be recorded instead of run). 28 tables of 128 KiB; a fill runs the operation's own
// functor over the 65 536 patterns.
hmr_status build_unary_tables(hmr_context &ctx) {
    Visit v;
    if (hmr_status s = v.use_device(ctx.device)) return s;
    void *block = nullptr;
    if (hmr_status s = v.hip(hipMalloc(&block, kTableSlots * kTableBytes + kCheckStateBytes), "hipMalloc(&tables, kTableSlots * kTableBytes)")) return s;
    char *state = static_cast<char *>(block) + kTableSlots * kTableBytes;
    (void)hipGetLastError();
    const auto fill = [&](auto t) {
        using T = typename decltype(t)::type;
        const int dtype = std::is_same_v<T, bf16_t> ? HMR_BF16 : HMR_F16;
        for (int op = kFirstTableOp; op <= kLastTableOp; ++op) {
            with_code(op, FloatOps{}, [&](auto o) {
                if constexpr (decltype(o)::value >= kFirstTableOp && decltype(o)::value <= kLastTableOp) {
                    using F = UnaryFloat<decltype(o)::value, T>;
                    launch_table_fill<F>(reinterpret_cast<uint16_t *>(static_cast<char *>(block) + table_slot(op, dtype) * kTableBytes),
                                         ctx.stream);
                }
            });
        }
    };
    fill(TypeTag<f16_t>{});
    fill(TypeTag<bf16_t>{});
    hipError_t ran = hipGetLastError();
    // The checks' meeting place: no bad position yet (all ones), no workgroup arrived.
    if (ran == hipSuccess) ran = hipMemsetAsync(state, 0, kCheckStateBytes, ctx.stream);
    if (ran == hipSuccess) ran = hipMemsetAsync(state, 0xFF, 8, ctx.stream);
    if (ran == hipSuccess) ran = hipStreamSynchronize(ctx.stream);
    if (ran != hipSuccess) {
        (void)hipFree(block);
        return v.hip(ran, "filling the tables of the 16-bit unary operations");
    }
    ctx.tables = block;
    ctx.check_state = state;
    return HMR_OK;
}

}  // namespace hmr

extern "C" hmr_status hmr_unary(hmr_context_t ctx, int32_t op, const hmr_tensor_desc *out,
                                const hmr_tensor_desc *src) {
    return hmr::fenced([&] {
        const hmr_tensor_desc *descs[2] = {out, src};
        return hmr::run_map(
            ctx, "unary", 2, descs, nullptr,
            [&](const hmr::MapCall &call, hipStream_t stream) {
                return hmr::pick_unary(ctx, op, out->dtype, src->dtype, call, stream);
            });
    });
}
