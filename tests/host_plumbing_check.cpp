// The library's host plumbing (homura_amd/csrc/runtime.hip, memory.hip, common.hpp) compiled as plain C++ against
// the scripted HIP of tests/fake_hip and driven through its failure paths: what a failing step of
// hmr_context_create leaves behind, the exception fence, the sticky last error, the caller's device, the armed
// test failures (ref: csrc/tests/host_failures.cpp does the same for the reference's plumbing; the contract is
// csrc/homura_rocm.h:1-15, 26-100, 612-626). Prints "host plumbing ok" and exits 0, or names the first failure.
#include <cstdio>
#include <string>
#include <thread>

#include "runtime.hip"
#include "memory.hip"

// The one function of the plumbing that lives beside device code (reduce.hip): the static block's address.
static int g_bind_calls = 0;
static bool g_bind_fails = false;
hmr_status hmr::bind_reduce_scratch(hmr_context &ctx) {
    ++g_bind_calls;
    if (g_bind_fails) return hmr::fail(HMR_HIP_ERROR, "hipGetSymbolAddress(&address, HIP_SYMBOL(scratch)): invalid resource handle");
    static unsigned char block[256];
    ctx.reduce_scratch = block;
    return HMR_OK;
}

static int g_released = 0;
void hmr::release_reduce_scratch(const hmr_context &) noexcept { ++g_released; }

// The other one (ew_unary.hip): the tables of the 16-bit unary operations. Here a block of the scripted HIP's
// memory, so that the books show who frees it.
static bool g_tables_fail = false;
hmr_status hmr::build_unary_tables(hmr_context &ctx) {
    if (g_tables_fail) return hmr::fail(HMR_OUT_OF_MEMORY, "hipMalloc(&tables, kTableSlots * kTableBytes): out of memory");
    void *block = nullptr;
    if (hipMalloc(&block, 64) != hipSuccess) return hmr::fail(HMR_OUT_OF_MEMORY, "hipMalloc(&tables, kTableSlots * kTableBytes): out of memory");
    ctx.tables = block;
    return HMR_OK;
}

// Large aligned copies and fills leave the plumbing for the kernels (ew_copy.hip, ew_misc.hip); here the calls
// are counted.
static int g_kernel_copies = 0, g_kernel_fills = 0;
static uint64_t g_fill_bits = 0;
extern "C" hmr_status hmr_copy(hmr_context_t, const hmr_tensor_desc *dst, const hmr_tensor_desc *src) {
    if (dst->ndim == 1 && src->ndim == 1 && dst->sizes[0] == src->sizes[0] && dst->dtype == src->dtype) ++g_kernel_copies;
    return HMR_OK;
}
extern "C" hmr_status hmr_fill(hmr_context_t, const hmr_tensor_desc *dst, uint64_t bits) {
    if (dst->ndim == 1) ++g_kernel_fills;
    g_fill_bits = bits;
    return HMR_OK;
}

static int g_failures = 0;
#define EXPECT(cond)                                                              \
    do {                                                                          \
        if (!(cond)) {                                                            \
            std::printf("line %d: %s   [last error: %s]\n", __LINE__, #cond, hmr_last_error()); \
            ++g_failures;                                                         \
        }                                                                         \
    } while (0)

static std::string last() { return hmr_last_error(); }
static fake::Machine &M() { return fake::machine(); }
static bool clean() {
    return M().streams.empty() && M().blocks.empty() && M().pinned.empty() && hmr_test_live_streams() == 0 && hipGetLastError() == hipSuccess;
}

static void devices() {
    int32_t n = -1;
    M().count_error = hipErrorNoDevice;
    EXPECT(hmr_device_count(&n) == HMR_OK && n == 0);
    EXPECT(hipGetLastError() == hipSuccess);  // a machine without GPUs leaves no error behind
    M().count_error = hipErrorInsufficientDriver;
    EXPECT(hmr_device_count(&n) == HMR_OK && n == 0);
    M().count_error = hipErrorInvalidValue;
    EXPECT(hmr_device_count(&n) == HMR_HIP_ERROR);
    EXPECT(hipGetLastError() == hipSuccess);
    M().count_error = hipSuccess;
    EXPECT(hmr_device_count(&n) == HMR_OK && n == 1);

    hmr_device_properties p;
    EXPECT(hmr_device_properties_get(1, &p) == HMR_INVALID && last() == "rocm:1 is not available: 1 ROCm device found");
    M().gpus.push_back(fake::Gpu{});
    EXPECT(hmr_device_properties_get(2, &p) == HMR_INVALID && last() == "rocm:2 is not available: 2 ROCm devices found");
    EXPECT(hmr_device_properties_get(-1, &p) == HMR_INVALID);
    EXPECT(hmr_device_properties_get(1, &p) == HMR_OK);
    EXPECT(std::string(p.arch) == "gfx950" && p.warp_size == 64 && p.multiprocessor_count == 256);
    EXPECT(std::string(p.name) == "AMD Instinct MI355X" && p.total_memory == (uint64_t{288} << 30));
    hmr_test_fail_properties(1);
    EXPECT(hmr_device_properties_get(0, &p) == HMR_HIP_ERROR);
    EXPECT(last() == "hipGetDeviceProperties(&p, device): invalid resource handle (injected for testing)");
    EXPECT(hmr_device_properties_get(0, &p) == HMR_OK);  // armed once
    uint64_t f = 0, t = 0;
    fake::thread().device = 1;
    EXPECT(hmr_mem_get_info(0, &f, &t) == HMR_OK && t == (uint64_t{288} << 30) && f == t / 2);
    EXPECT(fake::thread().device == 1);  // the caller's device is put back
    EXPECT(hmr_mem_get_info(5, &f, &t) == HMR_INVALID);
    fake::thread().device = 0;
}

static void contexts() {
    hmr_context_t ctx = reinterpret_cast<hmr_context_t>(0x1);
    // GPUs the library cannot drive.
    M().gpus[1].arch = "gfx1201";
    EXPECT(hmr_context_create(1, &ctx) == HMR_INVALID && ctx == nullptr);
    EXPECT(last() == "rocm:1 is a gfx1201 GPU, but homura was built for gfx950; rebuild it with HOMURA_OFFLOAD_ARCH set to "
                     "include gfx1201 (if homura supports it)");
    M().gpus[1].arch = "gfx950";
    M().gpus[1].wave = 32;
    EXPECT(hmr_context_create(1, &ctx) == HMR_INVALID && last() == "rocm:1 has a wave size of 32; this build of homura needs wave64");
    EXPECT(hmr_context_create(7, &ctx) == HMR_INVALID && last() == "rocm:7 is not available: 2 ROCm devices found");
    EXPECT(clean());
    M().gpus[1].wave = 64;

    // Every step that can fail, in order; each leaves nothing behind and the caller's device in place.
    fake::thread().device = 1;
    hmr_test_fail_stream_create(1);
    EXPECT(hmr_context_create(0, &ctx) == HMR_OUT_OF_MEMORY && ctx == nullptr);
    EXPECT(last() == "hipStreamCreateWithFlags(&s, hipStreamNonBlocking): out of memory (injected for testing)");
    EXPECT(clean() && fake::thread().device == 1);

    M().fail_next["hipStreamCreateWithFlags"] = hipErrorOutOfMemory;
    EXPECT(hmr_context_create(0, &ctx) == HMR_OUT_OF_MEMORY);
    EXPECT(last() == "hipStreamCreateWithFlags(&s, hipStreamNonBlocking): out of memory");
    EXPECT(clean() && fake::thread().device == 1);

    M().fail_next["hipMalloc"] = hipErrorOutOfMemory;  // the probe's buffer
    EXPECT(hmr_context_create(0, &ctx) == HMR_OUT_OF_MEMORY && last() == "rocm:0: hipMalloc(probe buffer): out of memory");
    EXPECT(clean());

    M().fail_next["launch"] = hipErrorLaunchFailure;
    EXPECT(hmr_context_create(0, &ctx) == HMR_HIP_ERROR);
    EXPECT(last() == "rocm:0: running the probe kernel: unspecified launch failure");
    EXPECT(clean());

    M().fail_next["hipStreamSynchronize"] = hipErrorLaunchFailure;
    EXPECT(hmr_context_create(0, &ctx) == HMR_HIP_ERROR && clean());

    // A GPU that reports 64 lanes but runs 32: the probe's upper half stays unwritten, and is noticed.
    M().gpus[0].lanes_run = 32;
    EXPECT(hmr_context_create(0, &ctx) == HMR_INTERNAL_ERROR && ctx == nullptr);
    EXPECT(last() == "rocm:0: the probe kernel wrote 0 in lane 32");
    EXPECT(clean() && fake::thread().device == 1);
    M().gpus[0].lanes_run = 0;

    // Success, and what a context owns.
    {
        hmr_context_t real = nullptr;
        EXPECT(hmr_context_create(0, &real) == HMR_OK && real != nullptr);
        EXPECT(hmr_test_live_streams() == 1 && M().streams.size() == 1 && M().blocks.size() == 1);  // its tables
        EXPECT(fake::thread().device == 1 && real->device == 0 && real->compute_units == 256 && real->reduce_scratch != nullptr);
        EXPECT(real->tables != nullptr && real->mailbox != nullptr && M().pinned.size() == 1);
        EXPECT(hmr_context_synchronize(real) == HMR_OK);
        M().fail_next["hipStreamSynchronize"] = hipErrorLaunchFailure;
        EXPECT(hmr_context_synchronize(real) == HMR_HIP_ERROR && last() == "hipStreamSynchronize(ctx->stream): unspecified launch failure");
        EXPECT(hipGetLastError() == hipSuccess);
        // Destroying frees the tables even when the stream will not go.
        M().fail_next["hipStreamDestroy"] = hipErrorInvalidHandle;
        const int released = g_released;
        EXPECT(hmr_context_destroy(real) == HMR_HIP_ERROR && last() == "hipStreamDestroy(ctx->stream): invalid resource handle");
        EXPECT(g_released == released + 1);  // the static reduction block goes back with the context
        EXPECT(M().blocks.empty() && M().pinned.empty());
        EXPECT(hmr_test_live_streams() == 1);  // the stream is still there, and still counted
        for (FakeStream *s : M().streams) delete s;  // the fake's books, for what follows
        M().streams.clear();
    }
    EXPECT(hmr_context_destroy(nullptr) == HMR_OK);

    // An exception after the probe (host memory runs out): the fence reports it, the stream is given back.
    const int live = hmr_test_live_streams();
    hmr_test_fail_after_probe(1);
    EXPECT(hmr_context_create(0, &ctx) == HMR_OUT_OF_MEMORY && ctx == nullptr && last() == "host allocation failed");
    EXPECT(hmr_test_live_streams() == live && M().streams.empty() && M().blocks.empty());

    g_bind_fails = true;
    EXPECT(hmr_context_create(0, &ctx) == HMR_HIP_ERROR && ctx == nullptr);
    EXPECT(hmr_test_live_streams() == live && M().streams.empty() && M().blocks.empty());
    g_bind_fails = false;

    // The tables cannot be had: the stream is given back, nothing stays allocated.
    g_tables_fail = true;
    EXPECT(hmr_context_create(0, &ctx) == HMR_OUT_OF_MEMORY && ctx == nullptr);
    EXPECT(hmr_test_live_streams() == live && M().streams.empty() && M().blocks.empty() && M().pinned.empty());
    g_tables_fail = false;

    // Nor the mailbox.
    M().fail_next["hipHostMalloc"] = hipErrorOutOfMemory;
    EXPECT(hmr_context_create(0, &ctx) == HMR_OUT_OF_MEMORY && ctx == nullptr && last() == "hipHostMalloc(&mailbox, 64): out of memory");
    EXPECT(hmr_test_live_streams() == live && M().streams.empty() && M().blocks.empty() && M().pinned.empty());
}

static void memory() {
    fake::thread().device = 1;
    hmr_context_t ctx = nullptr;
    EXPECT(hmr_context_create(0, &ctx) == HMR_OK);
    void *p = reinterpret_cast<void *>(0x1);
    M().fail_next["hipMalloc"] = hipErrorOutOfMemory;
    EXPECT(hmr_malloc(0, 1 << 20, &p) == HMR_OUT_OF_MEMORY && p == nullptr && last() == "hipMalloc(&p, nbytes): out of memory");
    EXPECT(hipGetLastError() == hipSuccess);  // not left behind for the next launch check
    EXPECT(hmr_malloc(0, 64, &p) == HMR_OK && p != nullptr && fake::thread().device == 1);
    void *nowhere = reinterpret_cast<void *>(0x1);
    EXPECT(hmr_malloc(9, 64, &nowhere) == HMR_HIP_ERROR && nowhere == nullptr);  // hipSetDevice refuses
    EXPECT(fake::thread().device == 1);

    void *d = nullptr;
    EXPECT(hmr_malloc(0, 16, &d) == HMR_OK);
    EXPECT(hmr_memset(ctx, d, 0x5A, 16) == HMR_OK);
    unsigned char host[16] = {0};
    EXPECT(hmr_copy_to_host(ctx, host, d, 16) == HMR_OK && host[0] == 0x5A && host[15] == 0x5A);
    // An armed failure fires before anything moves, once per armed count, with the status asked for.
    const unsigned char other[16] = {1, 2, 3};
    hmr_test_fail_data(2, 1);
    EXPECT(hmr_copy_from_host(ctx, d, other, 16) == HMR_OUT_OF_MEMORY && last() == "hipMemcpyAsync(HostToDevice): out of memory");
    EXPECT(hmr_copy_device(ctx, d, d, 16) == HMR_OUT_OF_MEMORY && last() == "hipMemcpyAsync(DeviceToDevice): out of memory");
    EXPECT(hmr_copy_to_host(ctx, host, d, 16) == HMR_OK && host[0] == 0x5A);
    hmr_test_fail_data(1, 0);
    EXPECT(hmr_copy_to_host(ctx, host, d, 16) == HMR_HIP_ERROR && last() == "hipMemcpyAsync(DeviceToHost): invalid resource handle");
    hmr_test_fail_data(0, 0);
    EXPECT(hmr_copy_from_host(ctx, d, other, 16) == HMR_OK);
    EXPECT(hmr_copy_to_host(ctx, host, d, 16) == HMR_OK && host[1] == 2);
    const size_t calls = M().calls.size();
    EXPECT(hmr_copy_device(ctx, d, d, 0) == HMR_OK && M().calls.size() == calls);  // nothing to do, nothing called
    // A read-back of what the mailbox mirrors is a wait and a host copy; any other transfer forgets the address.
    {
        const size_t before = M().calls.size();
        std::memcpy(ctx->mailbox, "\x11\x22\x33\x44\x55\x66\x77\x88" "ABCDEFGH", 16);
        ctx->mail_src = d;
        unsigned char got[16] = {0};
        EXPECT(hmr_copy_to_host(ctx, got, d, 16) == HMR_OK && got[0] == 0x11 && got[15] == 'H');
        bool copied = false;
        for (size_t k = before; k < M().calls.size(); ++k) copied = copied || M().calls[k] == "hipMemcpyAsync";
        EXPECT(!copied && ctx->mail_src == d);
        EXPECT(hmr_copy_to_host(ctx, got, d, 8) == HMR_OK && got[7] == 0x88);
        // With a ticket out, the read-back watches the mailbox for it: once it is there no HIP call is made at
        // all; while it is not, the read-back falls back to the wait on the stream after a tenth of a millisecond.
        ctx->mail_ticket = 7;
        static_cast<uint64_t *>(ctx->mailbox)[2] = 7;
        auto waits_since = [&](size_t from) {
            size_t n = 0;
            for (size_t k = from; k < M().calls.size(); ++k) n += M().calls[k] == "hipStreamSynchronize" || M().calls[k] == "hipMemcpyAsync";
            return n;
        };
        size_t mark = M().calls.size();
        EXPECT(hmr_copy_to_host(ctx, got, d, 16) == HMR_OK && got[8] == 'A' && waits_since(mark) == 0);
        ctx->mail_ticket = 8;
        mark = M().calls.size();
        EXPECT(hmr_copy_to_host(ctx, got, d, 16) == HMR_OK && waits_since(mark) == 1);
        ctx->mail_ticket = 0;
        EXPECT(hmr_copy_from_host(ctx, d, got, 8) == HMR_OK && ctx->mail_src == nullptr);
        ctx->mail_src = d;
        EXPECT(hmr_memset(ctx, d, 0, 16) == HMR_OK && ctx->mail_src == nullptr);
    }
    // A megabyte and more at aligned addresses goes to the kernels: words of eight bytes when they divide the
    // size, bytes otherwise; an armed failure still comes first.
    {
        void *big = reinterpret_cast<void *>(uintptr_t{1} << 40);
        EXPECT(hmr_copy_device(ctx, big, big, 1 << 20) == HMR_OK && g_kernel_copies == 1);
        EXPECT(hmr_copy_device(ctx, big, big, (1 << 20) + 3) == HMR_OK && g_kernel_copies == 2);
        hmr_test_fail_data(1, 1);
        EXPECT(hmr_copy_device(ctx, big, big, 1 << 20) == HMR_OUT_OF_MEMORY && g_kernel_copies == 2);
        EXPECT(hmr_memset(ctx, big, 0x5A, 1 << 20) == HMR_OK && g_kernel_fills == 1 && g_fill_bits == UINT64_C(0x5A5A5A5A5A5A5A5A));
        EXPECT(hmr_memset(ctx, big, 0x5A, (1 << 20) + 1) == HMR_OK && g_kernel_fills == 2 && g_fill_bits == 0x5A);
    }
    // The launch bracket: an armed failure, a kernel-less call, a launch that HIP refuses.
    hmr_test_fail_data(1, 0);
    bool queued = false;
    EXPECT(hmr::queue_on(ctx, "thing", [&](hipStream_t) { queued = true; return true; }) == HMR_HIP_ERROR && !queued);
    EXPECT(last() == "hipGetLastError(): invalid resource handle");
    EXPECT(hmr::queue_on(ctx, "thing", [&](hipStream_t) { return false; }) == HMR_INVALID && last() == "thing: unsupported dtype");
    EXPECT(hmr::queue_on(ctx, "thing", [&](hipStream_t s) { M().fail_next["launch"] = hipErrorLaunchFailure; hipLaunchKernelGGL(+[](int) {}, dim3(1), dim3(1), 0, s, 0); return true; }) == HMR_HIP_ERROR);
    EXPECT(last() == "hipGetLastError(): unspecified launch failure" && hipGetLastError() == hipSuccess);
    EXPECT(fake::thread().device == 1);

    void *stream = nullptr;
    EXPECT(hmr_ext_stream(ctx, &stream) == HMR_OK && stream == static_cast<void *>(ctx->stream));
    EXPECT(hmr_ext_stream(nullptr, &stream) == HMR_INVALID);
    EXPECT(hmr_free(0, d) == HMR_OK && hmr_free(0, p) == HMR_OK && hmr_free(0, nullptr) == HMR_OK);
    EXPECT(hmr_free(0, reinterpret_cast<void *>(0x40)) == HMR_HIP_ERROR);
    EXPECT(hmr_context_destroy(ctx) == HMR_OK && M().streams.empty() && M().blocks.empty());
    fake::thread().device = 0;
}

static void fence_and_threads() {
    EXPECT(hmr_test_fail("a message of this thread") == HMR_INVALID && last() == "a message of this thread");
    std::string theirs;
    int their_streams = -1;
    std::thread([&] {
        (void)hmr_test_fail("another thread's");
        hmr_context_t c = nullptr;
        (void)hmr_context_create(0, &c);
        their_streams = hmr_test_live_streams();
        theirs = hmr_test_fail("another thread's") == HMR_INVALID ? hmr_last_error() : "?";
        (void)hmr_context_destroy(c);
    }).join();
    EXPECT(theirs == "another thread's" && their_streams == 1);
    EXPECT(last() == "a message of this thread");  // untouched by the other thread
    EXPECT(hmr::fenced([]() -> hmr_status { throw std::runtime_error("boom"); }) == HMR_INTERNAL_ERROR && last() == "internal error: boom");
    EXPECT(hmr::fenced([]() -> hmr_status { throw 7; }) == HMR_INTERNAL_ERROR && last() == "internal error: unknown exception");
    EXPECT(hmr::fenced([]() -> hmr_status { throw std::bad_alloc(); }) == HMR_OUT_OF_MEMORY && last() == "host allocation failed");
    hmr_abi_info info;
    hmr_abi_check(&info);
    EXPECT(info.desc_size == 424 && info.max_dims == 25 && info.status_values[4] == HMR_INTERNAL_ERROR && info.dtype_values[9] == HMR_F64);
    EXPECT(std::string(hmr_built_archs()) == "gfx950");
    int32_t dev = -1;
    EXPECT(hmr_test_set_current_device(1) == HMR_OK && hmr_test_current_device(&dev) == HMR_OK && dev == 1);
    EXPECT(hmr_test_set_current_device(0) == HMR_OK);
}

int main() {
    devices();
    contexts();
    memory();
    fence_and_threads();
    if (g_failures == 0) std::printf("host plumbing ok\n");
    return g_failures == 0 ? 0 : 1;
}
