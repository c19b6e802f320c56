// What every translation unit of the library shares: the context, the calling thread's failure text and
// `Visit`, the object that stands for one entry point's stay inside the library.
//
// The contract these serve is the C ABI's (ref: csrc/homura_rocm.h:1-15): a status per call, a message that
// belongs to the calling thread, no C++ exception across the boundary, the caller's current device put back,
// and no failed HIP call left behind in hipGetLastError.
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
    int device = -1;
    hipStream_t stream = nullptr;
    int compute_units = 256;  // multiProcessorCount of the device (256 on MI355X), for grid sizing
    // Result tables of the 16-bit unary operations (one 128 KiB table per operation and dtype, every
    // input pattern -> its output pattern): allocated and filled by hmr_context_create, read-only afterwards,
    // freed with the context.
    void *tables = nullptr;
    // Where a position check spread over many workgroups meets (index.hip): the smallest bad position so far and
    // the count of workgroups that have finished. Device memory behind the tables; the last workgroup of a check
    // leaves both as it found them (all ones, zero).
    void *check_state = nullptr;
    // The mailbox: pinned host memory the GPU can write (three words in use). A kernel whose result the caller is
    // about to read back (the verdict of a position check) stores it there as well as in the caller's device
    // memory, and after it the ticket the launch was given (`mail_ticket`, counted up per check); `mail_src` is
    // that device address while the mailbox holds its current contents, and a read-back of it (hmr_copy_to_host)
    // watches the mailbox for the ticket - briefly, then it waits for the stream like any copy - and takes the
    // bytes from there instead of queueing a copy. Anything else queued on the context forgets the address.
    // Like the rest of a context these are the submitting thread's: the caller serialises its submissions per
    // device (the reference's execution mutex), and a read-back follows its check on the same thread.
    void *mailbox = nullptr;
    const void *mail_src = nullptr;
    uint64_t mail_ticket = 0;
    // Device address, on this context's GPU, of the library's static block for partial results
    // (hmr_reduce_static). Each GPU holds its own copy of the block at its own address.
    void *reduce_scratch = nullptr;
};

namespace hmr {

// ---- failures ------------------------------------------------------------------------------------------

// Makes `message` the calling thread's failure text and hands `status` back, so that a failure reads
// `return fail(HMR_INVALID, "...")`.
hmr_status fail(hmr_status status, std::string message);

// The same for a string literal. Nothing is allocated, so it works when memory is what ran out.
hmr_status fail_static(hmr_status status, const char *message) noexcept;

const char *last_error_text() noexcept;

// The failure of a HIP call as a status: out of memory is its own status, anything else HMR_HIP_ERROR, the
// text "<what>: <HIP's description>". HIP keeps the last error per thread until it is read; it is read here,
// so that the check after a later launch does not meet this failure again.
hmr_status hip_failure(hipError_t error, const char *what) noexcept;

// Looks up where the static block of hmr_reduce_static lives on the current device and keeps the address
// in the context. Called once per context, with its device current (defined beside the block, reduce.hip).
hmr_status bind_reduce_scratch(hmr_context &ctx);
// Gives the static block back if `ctx` is the context that holds it (hmr_context_destroy).
void release_reduce_scratch(const hmr_context &ctx) noexcept;

// Allocates the tables of the 16-bit unary operations on the context's GPU (and, behind them, the meeting place
// of the position checks), fills them on its stream and waits for the fills. Called once per context, after its
// stream exists (defined beside the operations, ew_unary.hip).
hmr_status build_unary_tables(hmr_context &ctx);
// Bytes kept behind the tables for hmr_context::check_state.
constexpr size_t kCheckStateBytes = 8192;

// ---- one entry point's stay in the library ---------------------------------------------------------------

class Visit {
  public:
    Visit() noexcept = default;
    Visit(const Visit &) = delete;
    Visit &operator=(const Visit &) = delete;
    // Leaves the calling thread on the device it came with.
    ~Visit() {
        if (moved_) (void)hipSetDevice(home_);
    }

    // Makes `device` current for the rest of the visit.
    hmr_status use_device(int device) noexcept {
        if (home_ < 0) {
            if (hmr_status s = hip(hipGetDevice(&home_), "hipGetDevice(&previous_)")) return s;
            now_ = home_;
        }
        if (device == now_) return HMR_OK;
        if (hmr_status s = hip(hipSetDevice(device), "hipSetDevice(device)")) return s;
        moved_ = true;
        now_ = device;
        return HMR_OK;
    }

    // HMR_OK for hipSuccess; otherwise the call's failure, recorded.
    hmr_status hip(hipError_t result, const char *what) noexcept {
        return result == hipSuccess ? HMR_OK : hip_failure(result, what);
    }

    // A test can arm the next data-moving steps of the calling thread to fail (hmr_test_fail_data). Each such
    // step asks here first, naming the HIP call it stands for, and fails the way that call would have.
    hmr_status armed_failure(const char *what) noexcept;

    // Queues one call's kernels on the context's stream. `queue(stream)` launches them and returns false,
    // having launched nothing, when it has no kernel for the dtype / operation. Around it: the device is made
    // current, an armed failure fires before anything is queued, HIP's last error is cleared and, afterwards,
    // read: that is where a launch that could not be queued shows.
    template <class Queue>
    hmr_status kernels(hmr_context_t ctx, const char *what, Queue queue) {
        if (ctx == nullptr) return fail(HMR_INVALID, std::string(what) + ": null context");
        ctx->mail_src = nullptr;  // whatever is queued may write what the mailbox mirrors
        if (hmr_status s = use_device(ctx->device)) return s;
        if (hmr_status s = armed_failure("hipGetLastError()")) return s;
        (void)hipGetLastError();
        if (!queue(ctx->stream)) return fail(HMR_INVALID, std::string(what) + ": unsupported dtype");
        return hip(hipGetLastError(), "hipGetLastError()");
    }

  private:
    int home_ = -1;  // the caller's device, once asked for
    int now_ = -1;   // the calling thread's current device
    bool moved_ = false;
};

// The exception fence of the C ABI: runs `body(visit)` with a fresh Visit and turns anything thrown into a
// status (a failed allocation of host memory is HMR_OUT_OF_MEMORY, the rest HMR_INTERNAL_ERROR).
template <class Body>
hmr_status visit(Body body) noexcept {
    try {
        Visit v;
        return body(v);
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

// The two forms most entry points need, for code that has no use for the Visit itself: the fence alone, and
// the kernels of one call (a Visit of its own; the device goes back when they are queued).
template <class Body>
hmr_status fenced(Body body) noexcept {
    return visit([&](Visit &) { return body(); });
}

template <class Queue>
hmr_status queue_on(hmr_context_t ctx, const char *what, Queue queue) {
    Visit v;
    return v.kernels(ctx, what, queue);
}

}  // namespace hmr
