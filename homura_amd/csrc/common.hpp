// Shared by every translation unit of the library: the context, the per-thread error channel,
// the exception fence of the C ABI and the current-device guard.
// Conventions follow ref: csrc/common.hpp:12-87 and csrc/homura_rocm.h:1-15.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>
#include <exception>
#include <mutex>
#include <new>
#include <string>

#include "homura_rocm.h"

// What hmr_context_t points at. One per device.
struct hmr_context {
    int device;
    hipStream_t stream;
    int compute_units;  // multiProcessorCount of the device (256 on MI355X), for grid sizing
    // Result tables of the 16-bit unary operations (one 128 KiB table per operation and dtype, every
    // input pattern -> its output pattern). The block is allocated at the first use and lives as long
    // as the context; a table is filled, on `stream`, by the first call that needs it.
    std::mutex table_lock;
    void *tables = nullptr;
    uint64_t tables_filled = 0;  // bit per table
    // Device address, on this context's GPU, of the library's static block for partial results
    // (hmr_reduce_static). Each GPU holds its own copy of the block at its own address.
    void *reduce_scratch = nullptr;
};

namespace hmr {

// Stores `message` as the calling thread's last error and hands `status` back.
hmr_status fail(hmr_status status, std::string message);

// Same for a string literal; allocates nothing, so it is safe where memory may be exhausted.
hmr_status fail_static(hmr_status status, const char *message) noexcept;

const char *last_error_text() noexcept;

// Reports a failed HIP call: out of memory maps to HMR_OUT_OF_MEMORY, everything else to
// HMR_HIP_ERROR. Also clears HIP's sticky per-thread error so that a later launch check does not
// see this failure again.
hmr_status hip_fail(hipError_t error, const char *call) noexcept;

#define HMR_HIP(expr)                                                         \
    do {                                                                      \
        hipError_t hmr_hip_e_ = (expr);                                       \
        if (hmr_hip_e_ != hipSuccess) return ::hmr::hip_fail(hmr_hip_e_, #expr); \
    } while (0)

// Looks up where the static block of hmr_reduce_static lives on the current device and keeps the address
// in the context. Called once per context, with its device current (defined beside the block, reduce.hip).
hmr_status bind_reduce_scratch(hmr_context &ctx);

// Consumes one failure armed by hmr_test_fail_data, if any: returns its status, else HMR_OK.
hmr_status injected_data_failure(const char *call) noexcept;

// Runs `body`; no exception gets past it.
template <class F>
hmr_status guarded(F body) noexcept {
    try {
        return body();
    } catch (const std::bad_alloc &) {
        return fail_static(HMR_OUT_OF_MEMORY, "host allocation failed");
    } catch (const std::exception &e) {
        try {
            return fail(HMR_INTERNAL_ERROR, std::string("internal error: ") + e.what());
        } catch (...) {
            return fail_static(HMR_INTERNAL_ERROR, "internal error (no memory for its message)");
        }
    } catch (...) {
        return fail_static(HMR_INTERNAL_ERROR, "internal error: unknown exception");
    }
}

// Makes `device` current for the calling thread and restores the previous device on scope exit.
class DeviceGuard {
  public:
    DeviceGuard() = default;
    DeviceGuard(const DeviceGuard &) = delete;
    DeviceGuard &operator=(const DeviceGuard &) = delete;
    ~DeviceGuard() {
        if (switched_) (void)hipSetDevice(previous_);
    }
    hmr_status enter(int device) {
        HMR_HIP(hipGetDevice(&previous_));
        if (previous_ != device) {
            HMR_HIP(hipSetDevice(device));
            switched_ = true;
        }
        return HMR_OK;
    }

  private:
    int previous_ = -1;
    bool switched_ = false;
};

// Brackets the launches `body(stream)` makes: device made current, an armed test failure fires
// before anything is queued, and hipGetLastError is checked afterwards. `body` returns false,
// having queued nothing, when it has no kernel for the dtype/op pair.
template <class F>
hmr_status launch_on(hmr_context_t ctx, const char *what, F body) {
    DeviceGuard guard;
    if (hmr_status s = guard.enter(ctx->device)) return s;
    if (hmr_status s = injected_data_failure("hipGetLastError()")) return s;
    (void)hipGetLastError();
    if (!body(ctx->stream)) return fail(HMR_INVALID, std::string(what) + ": unsupported dtype");
    HMR_HIP(hipGetLastError());
    return HMR_OK;
}

}  // namespace hmr
