// Error state, device queries, contexts, the ABI self-description and the test hooks.
// Behaviour follows ref: csrc/runtime.hip:132-379, re-targeted at gfx950 / 64-lane wavefronts
// (the reference refuses anything but wave32, ref: csrc/runtime.hip:257-260).
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

// Per thread: the last error (either an owned string or a literal) ...
thread_local std::string t_message;
thread_local const char *t_literal = nullptr;
// ... and the armed test failures plus the streams this thread holds.
thread_local int t_fail_stream = 0;
thread_local int t_fail_late = 0;
thread_local int t_fail_properties = 0;
thread_local int t_fail_data = 0;
thread_local bool t_fail_data_oom = false;
thread_local int t_streams = 0;

std::string arch_of(const hipDeviceProp_t &p) {
    std::string full(p.gcnArchName);
    return full.substr(0, full.find(':'));
}

bool arch_is_built(const std::string &arch) {
    const std::string list = HMR_OFFLOAD_ARCHS;
    size_t at = 0;
    for (;;) {
        size_t end = list.find(';', at);
        std::string item = list.substr(at, end == std::string::npos ? std::string::npos : end - at);
        if (item == arch) return true;
        if (end == std::string::npos) return false;
        at = end + 1;
    }
}

hmr_status device_in_range(int device) {
    int count = 0;
    HMR_HIP(hipGetDeviceCount(&count));
    if (device >= 0 && device < count) return HMR_OK;
    return fail(HMR_INVALID, "rocm:" + std::to_string(device) + " is not available: " + std::to_string(count) +
                                 " ROCm device" + (count == 1 ? "" : "s") + " found");
}

// A stream that is destroyed unless handed over; keeps the thread's live-stream count honest.
struct StreamHolder {
    hipStream_t stream = nullptr;
    StreamHolder() = default;
    StreamHolder(const StreamHolder &) = delete;
    StreamHolder &operator=(const StreamHolder &) = delete;
    ~StreamHolder() {
        if (stream) (void)drop(stream);
    }
    static hipError_t drop(hipStream_t s) noexcept {
        hipError_t e = hipStreamDestroy(s);
        if (e == hipSuccess) --t_streams;
        else (void)hipGetLastError();
        return e;
    }
    hmr_status open() {
        hipStream_t s = nullptr;
        HMR_HIP(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));
        stream = s;
        ++t_streams;
        return HMR_OK;
    }
    hipStream_t take() {
        hipStream_t s = stream;
        stream = nullptr;
        return s;
    }
};

constexpr uint32_t kProbeWord = 0x686d7264u;

// One wave writes lane-dependent words; lane 63 only exists on a 64-lane wavefront.
__global__ void probe_kernel(uint32_t *out) { out[threadIdx.x] = kProbeWord ^ threadIdx.x; }

// Proves at context creation that this library's code objects load and run on the GPU.
hmr_status run_probe(hipStream_t stream) {
    uint32_t *dev = nullptr;
    HMR_HIP(hipMalloc(&dev, 64 * sizeof(uint32_t)));
    uint32_t host[64] = {0};
    (void)hipGetLastError();
    hipLaunchKernelGGL(probe_kernel, dim3(1), dim3(64), 0, stream, dev);
    hipError_t e = hipGetLastError();
    if (e == hipSuccess) e = hipMemcpyAsync(host, dev, sizeof host, hipMemcpyDeviceToHost, stream);
    if (e == hipSuccess) e = hipStreamSynchronize(stream);
    hipError_t freed = hipFree(dev);
    if (e != hipSuccess) return hip_fail(e, "running the probe kernel");
    if (freed != hipSuccess) return hip_fail(freed, "hipFree(probe buffer)");
    for (uint32_t lane = 0; lane < 64; ++lane) {
        if (host[lane] != (kProbeWord ^ lane)) {
            return fail(HMR_INTERNAL_ERROR, "the probe kernel wrote " + std::to_string(host[lane]) + " in lane " +
                                                std::to_string(lane));
        }
    }
    return HMR_OK;
}

}  // namespace

hmr_status fail(hmr_status status, std::string message) {
    t_message = std::move(message);
    t_literal = nullptr;
    return status;
}

hmr_status fail_static(hmr_status status, const char *message) noexcept {
    t_literal = message;
    return status;
}

const char *last_error_text() noexcept { return t_literal ? t_literal : t_message.c_str(); }

hmr_status hip_fail(hipError_t error, const char *call) noexcept {
    (void)hipGetLastError();
    hmr_status status = error == hipErrorOutOfMemory ? HMR_OUT_OF_MEMORY : HMR_HIP_ERROR;
    try {
        return fail(status, std::string(call) + ": " + hipGetErrorString(error));
    } catch (...) {
        return fail_static(status, hipGetErrorString(error));
    }
}

hmr_status injected_data_failure(const char *call) noexcept {
    if (t_fail_data <= 0) return HMR_OK;
    --t_fail_data;
    return hip_fail(t_fail_data_oom ? hipErrorOutOfMemory : hipErrorInvalidHandle, call);
}

}  // namespace hmr

using hmr::fail;
using hmr::guarded;

extern "C" {

const char *hmr_last_error(void) { return hmr::last_error_text(); }

hmr_status hmr_device_count(int32_t *count) {
    return guarded([&] {
        int n = 0;
        hipError_t e = hipGetDeviceCount(&n);
        if (e == hipErrorNoDevice || e == hipErrorInsufficientDriver) {
            (void)hipGetLastError();
            n = 0;
        } else {
            HMR_HIP(e);
        }
        *count = n;
        return HMR_OK;
    });
}

hmr_status hmr_device_properties_get(int32_t device, hmr_device_properties *out) {
    return guarded([&] {
        if (hmr_status s = hmr::device_in_range(device)) return s;
        if (hmr::t_fail_properties > 0) {
            --hmr::t_fail_properties;
            return fail(HMR_HIP_ERROR,
                        "hipGetDeviceProperties(&p, device): invalid resource handle (injected for testing)");
        }
        hipDeviceProp_t p;
        HMR_HIP(hipGetDeviceProperties(&p, device));
        std::memset(out, 0, sizeof *out);
        std::strncpy(out->name, p.name, HMR_NAME_LEN - 1);
        std::strncpy(out->arch, hmr::arch_of(p).c_str(), HMR_ARCH_LEN - 1);
        out->multiprocessor_count = p.multiProcessorCount;
        out->warp_size = p.warpSize;
        out->total_memory = p.totalGlobalMem;
        return HMR_OK;
    });
}

hmr_status hmr_mem_get_info(int32_t device, uint64_t *free_bytes, uint64_t *total_bytes) {
    return guarded([&] {
        if (hmr_status s = hmr::device_in_range(device)) return s;
        hmr::DeviceGuard guard;
        if (hmr_status s = guard.enter(device)) return s;
        size_t f = 0, t = 0;
        HMR_HIP(hipMemGetInfo(&f, &t));
        *free_bytes = f;
        *total_bytes = t;
        return HMR_OK;
    });
}

hmr_status hmr_context_create(int32_t device, hmr_context_t *out) {
    return guarded([&] {
        *out = nullptr;
        if (hmr_status s = hmr::device_in_range(device)) return s;
        hipDeviceProp_t p;
        HMR_HIP(hipGetDeviceProperties(&p, device));
        std::string arch = hmr::arch_of(p);
        if (!hmr::arch_is_built(arch)) {
            return fail(HMR_INVALID, "rocm:" + std::to_string(device) + " is a " + arch +
                                         " GPU, but homura was built for " HMR_OFFLOAD_ARCHS
                                         "; rebuild it with HOMURA_OFFLOAD_ARCH set to include " +
                                         arch + " (if homura supports it)");
        }
        if (p.warpSize != 64) {
            return fail(HMR_INVALID, "rocm:" + std::to_string(device) + " has a wave size of " +
                                         std::to_string(p.warpSize) + "; this build of homura needs wave64");
        }
        // Host memory first, device resources after: any failure below unwinds cleanly.
        auto ctx = std::make_unique<hmr_context>();
        hmr::DeviceGuard guard;
        if (hmr_status s = guard.enter(device)) return s;
        hmr::StreamHolder holder;
        if (hmr::t_fail_stream > 0) {
            --hmr::t_fail_stream;
            return fail(HMR_OUT_OF_MEMORY,
                        "hipStreamCreateWithFlags(&s, hipStreamNonBlocking): out of memory (injected for testing)");
        }
        if (hmr_status s = holder.open()) return s;
        if (hmr_status s = hmr::run_probe(holder.stream)) {
            try {
                return fail(s, "rocm:" + std::to_string(device) + ": " + hmr::last_error_text());
            } catch (const std::bad_alloc &) {
                return s;
            }
        }
        if (hmr::t_fail_late > 0) {
            --hmr::t_fail_late;
            throw std::bad_alloc();
        }
        if (hmr_status s = hmr::bind_reduce_scratch(*ctx)) return s;
        ctx->device = device;
        ctx->compute_units = p.multiProcessorCount > 0 ? p.multiProcessorCount : 256;
        ctx->stream = holder.take();
        *out = ctx.release();
        return HMR_OK;
    });
}

hmr_status hmr_context_destroy(hmr_context_t ctx) {
    return guarded([&] {
        if (!ctx) return HMR_OK;
        hmr::DeviceGuard guard;
        if (hmr_status s = guard.enter(ctx->device)) return s;
        std::unique_ptr<hmr_context> owned(ctx);
        hipError_t e = hmr::StreamHolder::drop(owned->stream);
        if (e != hipSuccess) return hmr::hip_fail(e, "hipStreamDestroy(ctx->stream)");
        if (owned->tables != nullptr) HMR_HIP(hipFree(owned->tables));  // waits for the device
        return HMR_OK;
    });
}

hmr_status hmr_context_synchronize(hmr_context_t ctx) {
    return guarded([&] {
        hmr::DeviceGuard guard;
        if (hmr_status s = guard.enter(ctx->device)) return s;
        HMR_HIP(hipStreamSynchronize(ctx->stream));
        return HMR_OK;
    });
}

const char *hmr_built_archs(void) { return HMR_OFFLOAD_ARCHS; }

void hmr_abi_check(hmr_abi_info *out) {
    hmr_abi_info info;
    std::memset(&info, 0, sizeof info);
    info.abi_info_size = sizeof(hmr_abi_info);
    info.properties_size = sizeof(hmr_device_properties);
    info.properties_align = alignof(hmr_device_properties);
    const uint32_t prop_offsets[5] = {
        offsetof(hmr_device_properties, name), offsetof(hmr_device_properties, arch),
        offsetof(hmr_device_properties, multiprocessor_count), offsetof(hmr_device_properties, warp_size),
        offsetof(hmr_device_properties, total_memory)};
    std::memcpy(info.properties_offsets, prop_offsets, sizeof prop_offsets);
    const int32_t statuses[5] = {HMR_OK, HMR_OUT_OF_MEMORY, HMR_INVALID, HMR_HIP_ERROR, HMR_INTERNAL_ERROR};
    std::memcpy(info.status_values, statuses, sizeof statuses);
    info.name_len = HMR_NAME_LEN;
    info.arch_len = HMR_ARCH_LEN;
    info.desc_size = sizeof(hmr_tensor_desc);
    info.desc_align = alignof(hmr_tensor_desc);
    const uint32_t desc_offsets[6] = {offsetof(hmr_tensor_desc, data),  offsetof(hmr_tensor_desc, offset),
                                      offsetof(hmr_tensor_desc, dtype), offsetof(hmr_tensor_desc, ndim),
                                      offsetof(hmr_tensor_desc, sizes), offsetof(hmr_tensor_desc, strides)};
    std::memcpy(info.desc_offsets, desc_offsets, sizeof desc_offsets);
    const int32_t dtypes[10] = {HMR_BOOL, HMR_U8,  HMR_I8,   HMR_I16, HMR_I32,
                                HMR_I64,  HMR_F16, HMR_BF16, HMR_F32, HMR_F64};
    std::memcpy(info.dtype_values, dtypes, sizeof dtypes);
    info.max_dims = HMR_MAX_DIMS;
    info.gemm_desc_size = sizeof(hmr_gemm_desc);
    info.gemm_desc_align = alignof(hmr_gemm_desc);
    *out = info;
}

void hmr_test_fail_stream_create(int32_t n) { hmr::t_fail_stream = n; }
void hmr_test_fail_after_probe(int32_t n) { hmr::t_fail_late = n; }
void hmr_test_fail_properties(int32_t n) { hmr::t_fail_properties = n; }
void hmr_test_fail_data(int32_t n, int32_t out_of_memory) {
    hmr::t_fail_data = n;
    hmr::t_fail_data_oom = out_of_memory != 0;
}
int32_t hmr_test_live_streams(void) { return hmr::t_streams; }

hmr_status hmr_test_current_device(int32_t *device) {
    return guarded([&] {
        int d = -1;
        HMR_HIP(hipGetDevice(&d));
        *device = d;
        return HMR_OK;
    });
}

hmr_status hmr_test_set_current_device(int32_t device) {
    return guarded([&] {
        HMR_HIP(hipSetDevice(device));
        return HMR_OK;
    });
}

hmr_status hmr_test_fail(const char *message) {
    return guarded([&] { return fail(HMR_INVALID, message); });
}

}  // extern "C"
