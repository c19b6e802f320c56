// The calling thread's state, device queries, contexts, the ABI's description of itself and the test hooks
// (ref: csrc/homura_rocm.h:26-79, 590-666 for what each entry point promises). Built for gfx950 and 64-lane
// wavefronts: a GPU of another architecture or wave size is refused when a context is created.
#include <cstddef>
#include <cstring>
#include <memory>
#include <string>

#include "common.hpp"
#include "homura_rocm_unbuilt.h"

#ifndef HMR_OFFLOAD_ARCHS
#define HMR_OFFLOAD_ARCHS "gfx950"
#endif

namespace hmr {
namespace {

// Everything the library keeps per thread, in one place: the text of the last failure (an owned string, or a
// literal when nothing may be allocated), the failures a test has armed, and how many streams the thread holds.
struct ThreadState {
    std::string text;
    const char *literal = nullptr;
    struct Armed {
        int stream_create = 0;
        int after_probe = 0;
        int properties = 0;
        int data = 0;
        bool data_is_oom = false;
    } armed;
    int live_streams = 0;
};

ThreadState &mine() {
    thread_local ThreadState state;
    return state;
}

// Takes one of `count` armed failures, if any are left.
bool take(int &count) {
    if (count <= 0) return false;
    --count;
    return true;
}

// ---- what a GPU is ----------------------------------------------------------------------------------------

// gcnArchName without its feature suffix: "gfx950:sramecc+:xnack-" -> "gfx950".
std::string architecture(const hipDeviceProp_t &p) {
    const char *name = p.gcnArchName;
    const char *colon = std::strchr(name, ':');
    return colon ? std::string(name, colon) : std::string(name);
}

// Whether `arch` is one of the ';'-separated architectures this library holds code for.
bool has_code_for(const std::string &arch) {
    const char *list = HMR_OFFLOAD_ARCHS;
    const size_t len = arch.size();
    for (const char *at = list; *at != '\0';) {
        const char *end = std::strchr(at, ';');
        const size_t item = end ? static_cast<size_t>(end - at) : std::strlen(at);
        if (item == len && std::memcmp(at, arch.data(), len) == 0) return true;
        if (!end) break;
        at = end + 1;
    }
    return false;
}

hmr_status visible(Visit &v, int device) {
    int count = 0;
    if (hmr_status s = v.hip(hipGetDeviceCount(&count), "hipGetDeviceCount(&count)")) return s;
    if (device >= 0 && device < count) return HMR_OK;
    return fail(HMR_INVALID, "rocm:" + std::to_string(device) + " is not available: " + std::to_string(count) +
                                 " ROCm device" + (count == 1 ? "" : "s") + " found");
}

// ---- the probe: code objects load and 64 lanes run ----------------------------------------------------------

constexpr uint32_t kProbeWord = 0x686d7264u;
constexpr uint32_t kProbeLanes = 64;

// One wave writes a word per lane; lanes 32..63 only exist on a 64-lane wavefront.
__global__ void probe_kernel(uint32_t *out) { out[threadIdx.x] = kProbeWord ^ threadIdx.x; }

hmr_status run_probe(Visit &v, hipStream_t stream) {
    uint32_t *words = nullptr;
    if (hmr_status s = v.hip(hipMalloc(&words, kProbeLanes * sizeof(uint32_t)), "hipMalloc(probe buffer)")) return s;
    uint32_t seen[kProbeLanes] = {0};
    (void)hipGetLastError();
    hipLaunchKernelGGL(probe_kernel, dim3(1), dim3(kProbeLanes), 0, stream, words);
    hipError_t ran = hipGetLastError();
    if (ran == hipSuccess) ran = hipMemcpyAsync(seen, words, sizeof seen, hipMemcpyDeviceToHost, stream);
    if (ran == hipSuccess) ran = hipStreamSynchronize(stream);
    const hipError_t freed = hipFree(words);  // whatever happened above
    if (hmr_status s = v.hip(ran, "running the probe kernel")) return s;
    if (hmr_status s = v.hip(freed, "hipFree(probe buffer)")) return s;
    for (uint32_t lane = 0; lane < kProbeLanes; ++lane) {
        if (seen[lane] == (kProbeWord ^ lane)) continue;
        return fail(HMR_INTERNAL_ERROR,
                    "the probe kernel wrote " + std::to_string(seen[lane]) + " in lane " + std::to_string(lane));
    }
    return HMR_OK;
}

// ---- a context being put together ----------------------------------------------------------------------------

// Holds what a context owns while hmr_context_create goes through its steps; whatever step fails (or throws),
// the destructor gives back what was acquired so far. `release()` hands the finished context to the caller.
class ContextParts {
  public:
    ContextParts() : ctx_(std::make_unique<hmr_context>()) {}  // host memory first: may throw, nothing to undo yet
    ContextParts(const ContextParts &) = delete;
    ContextParts &operator=(const ContextParts &) = delete;
    ~ContextParts() {
        if (ctx_ && ctx_->tables != nullptr && hipFree(ctx_->tables) != hipSuccess) (void)hipGetLastError();
        if (ctx_ && ctx_->mailbox != nullptr && hipHostFree(ctx_->mailbox) != hipSuccess) (void)hipGetLastError();
        if (ctx_ && ctx_->stream != nullptr) (void)close(ctx_->stream);
    }

    hmr_context &ctx() { return *ctx_; }

    hmr_status open_stream(Visit &v) {
        if (take(mine().armed.stream_create)) {
            return fail(HMR_OUT_OF_MEMORY,
                        "hipStreamCreateWithFlags(&s, hipStreamNonBlocking): out of memory (injected for testing)");
        }
        hipStream_t s = nullptr;
        if (hmr_status e = v.hip(hipStreamCreateWithFlags(&s, hipStreamNonBlocking),
                                 "hipStreamCreateWithFlags(&s, hipStreamNonBlocking)")) {
            return e;
        }
        ctx_->stream = s;
        ++mine().live_streams;
        return HMR_OK;
    }

    // The mailbox: pinned host memory that kernels on this GPU may write.
    hmr_status open_mailbox(Visit &v) {
        void *box = nullptr;
        if (hmr_status e = v.hip(hipHostMalloc(&box, 64, hipHostMallocDefault), "hipHostMalloc(&mailbox, 64)")) return e;
        std::memset(box, 0, 64);
        ctx_->mailbox = box;
        return HMR_OK;
    }

    hmr_context *release() { return ctx_.release(); }

    // Destroys a stream and keeps the thread's count of live streams right.
    static hipError_t close(hipStream_t stream) noexcept {
        const hipError_t e = hipStreamDestroy(stream);
        if (e == hipSuccess) --mine().live_streams;
        else (void)hipGetLastError();
        return e;
    }

  private:
    std::unique_ptr<hmr_context> ctx_;
};

}  // namespace

// ---- failures (declared in common.hpp) -------------------------------------------------------------------------

hmr_status fail(hmr_status status, std::string message) {
    ThreadState &t = mine();
    t.text = std::move(message);
    t.literal = nullptr;
    return status;
}

hmr_status fail_static(hmr_status status, const char *message) noexcept {
    mine().literal = message;
    return status;
}

const char *last_error_text() noexcept {
    const ThreadState &t = mine();
    return t.literal ? t.literal : t.text.c_str();
}

hmr_status hip_failure(hipError_t error, const char *what) noexcept {
    (void)hipGetLastError();
    const hmr_status status = error == hipErrorOutOfMemory ? HMR_OUT_OF_MEMORY : HMR_HIP_ERROR;
    const char *description = hipGetErrorString(error);
    try {
        return fail(status, std::string(what) + ": " + description);
    } catch (...) {
        return fail_static(status, description);
    }
}

hmr_status Visit::armed_failure(const char *what) noexcept {
    ThreadState::Armed &armed = mine().armed;
    if (!take(armed.data)) return HMR_OK;
    return hip_failure(armed.data_is_oom ? hipErrorOutOfMemory : hipErrorInvalidHandle, what);
}

}  // namespace hmr

using hmr::fail;
using hmr::Visit;

extern "C" {

const char *hmr_last_error(void) { return hmr::last_error_text(); }

hmr_status hmr_device_count(int32_t *count) {
    return hmr::visit([&](Visit &v) {
        int found = 0;
        const hipError_t e = hipGetDeviceCount(&found);
        if (e == hipErrorNoDevice || e == hipErrorInsufficientDriver) {
            (void)hipGetLastError();  // a machine without a GPU or a driver has zero devices; that is no failure
            *count = 0;
            return HMR_OK;
        }
        if (hmr_status s = v.hip(e, "hipGetDeviceCount(&n)")) return s;
        *count = found;
        return HMR_OK;
    });
}

hmr_status hmr_device_properties_get(int32_t device, hmr_device_properties *out) {
    return hmr::visit([&](Visit &v) {
        if (hmr_status s = hmr::visible(v, device)) return s;
        if (hmr::take(hmr::mine().armed.properties)) {
            return fail(HMR_HIP_ERROR,
                        "hipGetDeviceProperties(&p, device): invalid resource handle (injected for testing)");
        }
        hipDeviceProp_t p;
        if (hmr_status s = v.hip(hipGetDeviceProperties(&p, device), "hipGetDeviceProperties(&p, device)")) return s;
        hmr_device_properties filled;
        std::memset(&filled, 0, sizeof filled);
        std::strncpy(filled.name, p.name, HMR_NAME_LEN - 1);
        std::strncpy(filled.arch, hmr::architecture(p).c_str(), HMR_ARCH_LEN - 1);
        filled.multiprocessor_count = p.multiProcessorCount;  // compute units on CDNA, as they are
        filled.warp_size = p.warpSize;
        filled.total_memory = p.totalGlobalMem;
        *out = filled;
        return HMR_OK;
    });
}

hmr_status hmr_mem_get_info(int32_t device, uint64_t *free_bytes, uint64_t *total_bytes) {
    return hmr::visit([&](Visit &v) {
        if (hmr_status s = hmr::visible(v, device)) return s;
        if (hmr_status s = v.use_device(device)) return s;
        size_t free_now = 0, total = 0;
        if (hmr_status s = v.hip(hipMemGetInfo(&free_now, &total), "hipMemGetInfo(&f, &t)")) return s;
        *free_bytes = free_now;
        *total_bytes = total;
        return HMR_OK;
    });
}

hmr_status hmr_context_create(int32_t device, hmr_context_t *out) {
    return hmr::visit([&](Visit &v) {
        *out = nullptr;
        // Is this a GPU the library can drive?
        if (hmr_status s = hmr::visible(v, device)) return s;
        hipDeviceProp_t p;
        if (hmr_status s = v.hip(hipGetDeviceProperties(&p, device), "hipGetDeviceProperties(&p, device)")) return s;
        const std::string arch = hmr::architecture(p);
        const std::string who = "rocm:" + std::to_string(device);
        if (!hmr::has_code_for(arch)) {
            return fail(HMR_INVALID, who + " is a " + arch + " GPU, but homura was built for " HMR_OFFLOAD_ARCHS
                                         "; rebuild it with HOMURA_OFFLOAD_ARCH set to include " + arch +
                                         " (if homura supports it)");
        }
        if (p.warpSize != 64) {
            return fail(HMR_INVALID, who + " has a wave size of " + std::to_string(p.warpSize) +
                                         "; this build of homura needs wave64");
        }
        // Put the context together; ContextParts takes back what a failing step leaves.
        hmr::ContextParts parts;
        if (hmr_status s = v.use_device(device)) return s;
        if (hmr_status s = parts.open_stream(v)) return s;
        if (hmr_status s = hmr::run_probe(v, parts.ctx().stream)) {
            try {
                return fail(s, who + ": " + hmr::last_error_text());
            } catch (const std::bad_alloc &) {
                return s;  // the probe's own message stands
            }
        }
        if (hmr::take(hmr::mine().armed.after_probe)) throw std::bad_alloc();
        if (hmr_status s = hmr::bind_reduce_scratch(parts.ctx())) return s;
        parts.ctx().device = device;
        parts.ctx().compute_units = p.multiProcessorCount > 0 ? p.multiProcessorCount : 256;
        if (hmr_status s = parts.open_mailbox(v)) return s;
        if (hmr_status s = hmr::build_unary_tables(parts.ctx())) return s;
        *out = parts.release();
        return HMR_OK;
    });
}

hmr_status hmr_context_destroy(hmr_context_t ctx) {
    return hmr::visit([&](Visit &v) {
        if (ctx == nullptr) return HMR_OK;
        if (hmr_status s = v.use_device(ctx->device)) return s;
        const std::unique_ptr<hmr_context> owned(ctx);
        hmr::release_reduce_scratch(*owned);
        // Both resources go whatever the first one's fate: the first failure is the one reported.
        const hipError_t stream_gone = hmr::ContextParts::close(owned->stream);
        const hipError_t tables_gone = owned->tables != nullptr ? hipFree(owned->tables) : hipSuccess;  // waits for the device
        const hipError_t mailbox_gone = owned->mailbox != nullptr ? hipHostFree(owned->mailbox) : hipSuccess;
        if (hmr_status s = v.hip(stream_gone, "hipStreamDestroy(ctx->stream)")) return s;
        if (hmr_status s = v.hip(tables_gone, "hipFree(ctx->tables)")) return s;
        return v.hip(mailbox_gone, "hipHostFree(ctx->mailbox)");
    });
}

hmr_status hmr_context_synchronize(hmr_context_t ctx) {
    return hmr::visit([&](Visit &v) {
        if (hmr_status s = v.use_device(ctx->device)) return s;
        return v.hip(hipStreamSynchronize(ctx->stream), "hipStreamSynchronize(ctx->stream)");
    });
}

const char *hmr_built_archs(void) { return HMR_OFFLOAD_ARCHS; }

// What the caller's bindings can check against their own declarations (ref: csrc/homura_rocm.h:592-610).
void hmr_abi_check(hmr_abi_info *out) {
    hmr_abi_info info;
    std::memset(&info, 0, sizeof info);
    info.abi_info_size = sizeof(hmr_abi_info);

    using P = hmr_device_properties;
    info.properties_size = sizeof(P);
    info.properties_align = alignof(P);
    info.properties_offsets[0] = offsetof(P, name);
    info.properties_offsets[1] = offsetof(P, arch);
    info.properties_offsets[2] = offsetof(P, multiprocessor_count);
    info.properties_offsets[3] = offsetof(P, warp_size);
    info.properties_offsets[4] = offsetof(P, total_memory);
    info.name_len = HMR_NAME_LEN;
    info.arch_len = HMR_ARCH_LEN;

    using D = hmr_tensor_desc;
    info.desc_size = sizeof(D);
    info.desc_align = alignof(D);
    info.desc_offsets[0] = offsetof(D, data);
    info.desc_offsets[1] = offsetof(D, offset);
    info.desc_offsets[2] = offsetof(D, dtype);
    info.desc_offsets[3] = offsetof(D, ndim);
    info.desc_offsets[4] = offsetof(D, sizes);
    info.desc_offsets[5] = offsetof(D, strides);
    info.max_dims = HMR_MAX_DIMS;

    const int32_t statuses[] = {HMR_OK, HMR_OUT_OF_MEMORY, HMR_INVALID, HMR_HIP_ERROR, HMR_INTERNAL_ERROR};
    for (int i = 0; i < 5; ++i) info.status_values[i] = statuses[i];
    const int32_t dtypes[] = {HMR_BOOL, HMR_U8, HMR_I8, HMR_I16, HMR_I32, HMR_I64, HMR_F16, HMR_BF16, HMR_F32, HMR_F64};
    for (int i = 0; i < 10; ++i) info.dtype_values[i] = dtypes[i];

    info.gemm_desc_size = sizeof(hmr_gemm_desc);
    info.gemm_desc_align = alignof(hmr_gemm_desc);
    *out = info;
}

// ---- test hooks (ref: csrc/homura_rocm.h:612-666; not part of the supported interface) --------------------------

void hmr_test_fail_stream_create(int32_t n) { hmr::mine().armed.stream_create = n; }
void hmr_test_fail_after_probe(int32_t n) { hmr::mine().armed.after_probe = n; }
void hmr_test_fail_properties(int32_t n) { hmr::mine().armed.properties = n; }
void hmr_test_fail_data(int32_t n, int32_t out_of_memory) {
    hmr::mine().armed.data = n;
    hmr::mine().armed.data_is_oom = out_of_memory != 0;
}
int32_t hmr_test_live_streams(void) { return hmr::mine().live_streams; }

hmr_status hmr_test_current_device(int32_t *device) {
    return hmr::visit([&](Visit &v) {
        int current = -1;
        if (hmr_status s = v.hip(hipGetDevice(&current), "hipGetDevice(&d)")) return s;
        *device = current;
        return HMR_OK;
    });
}

hmr_status hmr_test_set_current_device(int32_t device) {
    return hmr::visit([&](Visit &v) { return v.hip(hipSetDevice(device), "hipSetDevice(device)"); });
}

hmr_status hmr_test_fail(const char *message) {
    return hmr::visit([&](Visit &) { return fail(HMR_INVALID, message); });
}

}  // extern "C"
