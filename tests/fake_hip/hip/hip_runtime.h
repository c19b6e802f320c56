// A scripted stand-in for the HIP runtime, for testing the library's host plumbing (homura_amd/csrc/runtime.hip,
// memory.hip) on a machine without a GPU: the same source files are compiled as plain C++ against this header.
// The test sets up GPUs, arms failures of particular HIP calls and inspects what the library left behind
// (streams, allocations, the current device, the sticky last error).
// The technique is the reference's (ref: csrc/tests/fake_hip/hip/hip_runtime.h, csrc/tests/host_failures.cpp);
// this header is written for this library's own plumbing.
#pragma once

#include <cstddef>
#include <cstdint>
#include <cstdlib>
#include <cstring>
#include <map>
#include <set>
#include <string>
#include <vector>

enum hipError_t {
    hipSuccess = 0,
    hipErrorInvalidValue = 1,
    hipErrorOutOfMemory = 2,
    hipErrorInsufficientDriver = 35,
    hipErrorNoDevice = 100,
    hipErrorInvalidDevice = 101,
    hipErrorInvalidHandle = 400,
    hipErrorLaunchFailure = 719,
};
enum hipMemcpyKind { hipMemcpyHostToDevice = 1, hipMemcpyDeviceToHost = 2, hipMemcpyDeviceToDevice = 3 };
constexpr unsigned hipStreamNonBlocking = 1;

struct hipDeviceProp_t {
    char name[256];
    char gcnArchName[256];
    int multiProcessorCount;
    int warpSize;
    size_t totalGlobalMem;
};
struct FakeStream {
    int device;
};
typedef FakeStream *hipStream_t;
struct dim3 {
    unsigned x, y, z;
    dim3(unsigned x_ = 1, unsigned y_ = 1, unsigned z_ = 1) : x(x_), y(y_), z(z_) {}
};
#define __global__
#define __device__
#define __host__
#define __forceinline__ inline
#define HIP_SYMBOL(x) (&(x))

namespace fake {

struct Gpu {
    std::string name = "AMD Instinct MI355X";
    std::string arch = "gfx950:sramecc+:xnack-";
    int compute_units = 256;
    int wave = 64;      // the wave size the GPU reports
    int lanes_run = 0;  // lanes of a block a launch really runs (0: as many as `wave`): a GPU that is not what it says
    size_t memory = size_t{288} << 30;
};

// The whole machine. `fail_next[name]` makes the next call of that HIP function return the given error.
struct Machine {
    std::vector<Gpu> gpus{Gpu{}};
    hipError_t count_error = hipSuccess;  // what hipGetDeviceCount reports instead of a count
    std::map<std::string, hipError_t> fail_next;
    std::set<void *> blocks;       // live device allocations
    std::set<void *> pinned;       // live pinned host allocations
    std::set<FakeStream *> streams;
    std::vector<std::string> calls;  // names of the HIP calls made, in order
};
inline Machine &machine() {
    static Machine m;
    return m;
}
struct Thread {
    int device = 0;
    hipError_t last = hipSuccess;
};
inline Thread &thread() {
    thread_local Thread t;
    return t;
}
inline hipError_t done(const char *name, hipError_t real = hipSuccess) {
    Machine &m = machine();
    m.calls.emplace_back(name);
    hipError_t e = real;
    auto armed = m.fail_next.find(name);
    if (armed != m.fail_next.end()) {
        e = armed->second;
        m.fail_next.erase(armed);
    }
    if (e != hipSuccess) thread().last = e;
    return e;
}
inline bool armed(const char *name) { return machine().fail_next.count(name) != 0; }
struct Index {
    unsigned x = 0;
};

}  // namespace fake

inline thread_local fake::Index threadIdx;

inline hipError_t hipGetLastError() {
    const hipError_t e = fake::thread().last;
    fake::thread().last = hipSuccess;
    return e;
}
inline const char *hipGetErrorString(hipError_t e) {
    switch (e) {
        case hipSuccess: return "no error";
        case hipErrorOutOfMemory: return "out of memory";
        case hipErrorInvalidHandle: return "invalid resource handle";
        case hipErrorNoDevice: return "no ROCm-capable device is detected";
        case hipErrorInvalidDevice: return "invalid device ordinal";
        case hipErrorLaunchFailure: return "unspecified launch failure";
        default: return "some other error";
    }
}
inline hipError_t hipGetDeviceCount(int *n) {
    if (fake::machine().count_error != hipSuccess) return fake::done("hipGetDeviceCount", fake::machine().count_error);
    *n = static_cast<int>(fake::machine().gpus.size());
    return fake::done("hipGetDeviceCount");
}
inline hipError_t hipGetDevice(int *d) {
    *d = fake::thread().device;
    return fake::done("hipGetDevice");
}
inline hipError_t hipSetDevice(int d) {
    if (d < 0 || d >= static_cast<int>(fake::machine().gpus.size())) return fake::done("hipSetDevice", hipErrorInvalidDevice);
    if (fake::armed("hipSetDevice")) return fake::done("hipSetDevice");
    fake::thread().device = d;
    return fake::done("hipSetDevice");
}
inline hipError_t hipGetDeviceProperties(hipDeviceProp_t *p, int d) {
    if (d < 0 || d >= static_cast<int>(fake::machine().gpus.size())) return fake::done("hipGetDeviceProperties", hipErrorInvalidDevice);
    const fake::Gpu &g = fake::machine().gpus[d];
    std::memset(p, 0, sizeof *p);
    std::strncpy(p->name, g.name.c_str(), sizeof p->name - 1);
    std::strncpy(p->gcnArchName, g.arch.c_str(), sizeof p->gcnArchName - 1);
    p->multiProcessorCount = g.compute_units;
    p->warpSize = g.wave;
    p->totalGlobalMem = g.memory;
    return fake::done("hipGetDeviceProperties");
}
inline hipError_t hipMemGetInfo(size_t *f, size_t *t) {
    *t = fake::machine().gpus[fake::thread().device].memory;
    *f = *t / 2;
    return fake::done("hipMemGetInfo");
}
inline hipError_t hipMalloc(void **p, size_t n) {
    if (fake::armed("hipMalloc")) return fake::done("hipMalloc");
    *p = std::calloc(n ? n : 1, 1);
    fake::machine().blocks.insert(*p);
    return fake::done("hipMalloc");
}
template <class T>
hipError_t hipMalloc(T **p, size_t n) {
    return hipMalloc(reinterpret_cast<void **>(p), n);
}
inline hipError_t hipFree(void *p) {
    if (p != nullptr) {
        if (!fake::machine().blocks.erase(p)) return fake::done("hipFree", hipErrorInvalidValue);
        std::free(p);
    }
    return fake::done("hipFree");
}
// Pinned host memory: its own book, so that a leak of it shows.
constexpr unsigned hipHostMallocDefault = 0;
inline hipError_t hipHostMalloc(void **p, size_t n, unsigned) {
    if (fake::armed("hipHostMalloc")) return fake::done("hipHostMalloc");
    *p = std::calloc(n ? n : 1, 1);
    fake::machine().pinned.insert(*p);
    return fake::done("hipHostMalloc");
}
inline hipError_t hipHostFree(void *p) {
    if (p != nullptr) {
        if (!fake::machine().pinned.erase(p)) return fake::done("hipHostFree", hipErrorInvalidValue);
        std::free(p);
    }
    return fake::done("hipHostFree");
}
inline hipError_t hipStreamCreateWithFlags(hipStream_t *s, unsigned) {
    if (fake::armed("hipStreamCreateWithFlags")) return fake::done("hipStreamCreateWithFlags");
    *s = new FakeStream{fake::thread().device};
    fake::machine().streams.insert(*s);
    return fake::done("hipStreamCreateWithFlags");
}
inline hipError_t hipStreamDestroy(hipStream_t s) {
    if (fake::armed("hipStreamDestroy")) return fake::done("hipStreamDestroy");
    if (!fake::machine().streams.erase(s)) return fake::done("hipStreamDestroy", hipErrorInvalidHandle);
    delete s;
    return fake::done("hipStreamDestroy");
}
inline hipError_t hipStreamSynchronize(hipStream_t) { return fake::done("hipStreamSynchronize"); }
inline hipError_t hipMemcpyAsync(void *dst, const void *src, size_t n, hipMemcpyKind, hipStream_t) {
    if (fake::armed("hipMemcpyAsync")) return fake::done("hipMemcpyAsync");
    std::memcpy(dst, src, n);
    return fake::done("hipMemcpyAsync");
}
inline hipError_t hipMemsetAsync(void *p, int value, size_t n, hipStream_t) {
    if (fake::armed("hipMemsetAsync")) return fake::done("hipMemsetAsync");
    std::memset(p, value, n);
    return fake::done("hipMemsetAsync");
}
// A launch runs the kernel on the host, once per lane the GPU really runs (so a GPU with 32-lane waves leaves the
// upper half of a 64-lane block unwritten), unless a launch failure is armed.
template <class Kernel, class... Args>
void fake_launch(Kernel kernel, dim3 block, hipStream_t stream, Args... args) {
    if (fake::armed("launch")) {
        (void)fake::done("launch");
        return;
    }
    const fake::Gpu &gpu = fake::machine().gpus[stream->device];
    const unsigned lanes = static_cast<unsigned>(gpu.lanes_run > 0 ? gpu.lanes_run : gpu.wave);
    for (unsigned lane = 0; lane < block.x && lane < lanes; ++lane) {
        threadIdx.x = lane;
        kernel(args...);
    }
    threadIdx.x = 0;
    (void)fake::done("launch");
}
#define hipLaunchKernelGGL(kernel, grid, block, shared, stream, ...) fake_launch(kernel, block, stream, __VA_ARGS__)
