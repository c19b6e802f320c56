// Compares homura_amd/csrc/expf_like_libm.hpp with the host library's expf over bit patterns of f32:
// `expf_check <stride> <fused 0|1>` walks every stride-th pattern (1: all 2^32) on all hardware threads and
// prints the number of inputs whose results differ in any bit (NaNs compare as equal).
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <thread>
#include <vector>

#include "expf_like_libm.hpp"

template <bool FUSED>
static uint64_t count(uint64_t begin, uint64_t end, uint64_t stride, uint32_t *first) {
    uint64_t bad = 0;
    for (uint64_t b = begin; b < end; b += stride) {
        const uint32_t bits = static_cast<uint32_t>(b);
        float x;
        memcpy(&x, &bits, 4);
        volatile float xv = x;  // keep the compiler from folding the library call
        const float want = expf(xv), got = hmr::expf_like_libm<FUSED>(x);
        uint32_t w, g;
        memcpy(&w, &want, 4);
        memcpy(&g, &got, 4);
        if (w != g && !(want != want && got != got)) {
            if (bad == 0) *first = bits;
            ++bad;
        }
    }
    return bad;
}

int main(int argc, char **argv) {
    const uint64_t stride = argc > 1 ? strtoull(argv[1], nullptr, 10) : 1;
    const bool fused = argc > 2 ? atoi(argv[2]) != 0 : true;
    const unsigned workers = std::max(1u, std::thread::hardware_concurrency());
    std::vector<uint64_t> bad(workers, 0);
    std::vector<uint32_t> first(workers, 0);
    std::vector<std::thread> pool;
    const uint64_t total = uint64_t{1} << 32, span = (total / workers / stride + 1) * stride;
    for (unsigned w = 0; w < workers; ++w) {
        pool.emplace_back([&, w] {
            const uint64_t begin = w * span, end = std::min(total, begin + span);
            bad[w] = fused ? count<true>(begin, end, stride, &first[w]) : count<false>(begin, end, stride, &first[w]);
        });
    }
    for (auto &t : pool) t.join();
    uint64_t sum = 0;
    uint32_t example = 0;
    for (unsigned w = 0; w < workers; ++w) {
        if (bad[w] && !sum) example = first[w];
        sum += bad[w];
    }
    std::printf("%llu differ", static_cast<unsigned long long>(sum));
    if (sum) std::printf(" (first at bits 0x%08x)", example);
    std::printf("\n");
    return 0;
}
