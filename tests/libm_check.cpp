// Compares the restated f32 library functions of homura_amd/csrc (expf_like_libm.hpp, f32_like_libm.hpp) with the
// host C library's over bit patterns of f32: `libm_check <function> <stride> [fused]` with function one of expf,
// expm1f, tanhf, log1pf, sinf, cosf, logf walks every stride-th pattern (1: all 2^32) on all hardware threads and prints the number of
// inputs whose results differ in any bit (a NaN for a NaN counts as equal); powf has two arguments and a mode of its
// own, the f64 functions tanh and expm1 are sampled (both below). `fused` (expf, sinf, cosf, logf; default 1)
// picks the form with fused multiply-adds.
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <thread>
#include <vector>

#include "expf_like_libm.hpp"
#include "f32_like_libm.hpp"
#include "sinf_cosf_logf_like_libm.hpp"
#include "powf_like_libm.hpp"
#include "f64_like_libm.hpp"

template <class Host, class Port>
static uint64_t count(uint64_t begin, uint64_t end, uint64_t stride, uint32_t *first, Host host, Port port) {
    uint64_t bad = 0;
    for (uint64_t b = begin; b < end; b += stride) {
        const uint32_t bits = static_cast<uint32_t>(b);
        float x;
        memcpy(&x, &bits, 4);
        volatile float xv = x;  // keep the compiler from folding the library call
        const float want = host(xv), got = port(x);
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

// powf: `libm_check powf <stride> [fused]` walks every stride-th base for each of 26 exponents, then
// 250 000 000 / stride * 8 random pairs (half of them with exponents that are multiples of 1/64).
template <bool FUSED>
static uint64_t powf_differences(uint64_t stride) {
    const float exponents[] = {0.5f, 2.0f, 3.0f, -1.0f, 1.0f / 3.0f, 0.1f, 2.5f, -0.5f, 7.0f, 1e-3f, 100.0f, -3.0f, 1.0f,
                               0.0f, -0.0f, INFINITY, -INFINITY, NAN, 1e-30f, 1e30f, 4.0f, 5.0f, 0.75f, -2.0f, 33.333f, 1.5f};
    const unsigned workers = std::max(1u, std::thread::hardware_concurrency());
    std::vector<uint64_t> bad(workers, 0);
    std::vector<std::thread> pool;
    auto differ = [](float x, float y) {
        volatile float xv = x, yv = y;
        const float want = powf(xv, yv), got = hmr::powf_like_libm<FUSED>(x, y);
        uint32_t w, g;
        memcpy(&w, &want, 4);
        memcpy(&g, &got, 4);
        return w != g && !(want != want && got != got);
    };
    for (unsigned w = 0; w < workers; ++w) {
        pool.emplace_back([&, w] {
            const uint64_t total = uint64_t{1} << 32, span = (total / workers / stride + 1) * stride;
            for (float y : exponents) {
                for (uint64_t b = w * span; b < std::min(total, (w + 1) * span); b += stride) {
                    const uint32_t bits = static_cast<uint32_t>(b);
                    float x;
                    memcpy(&x, &bits, 4);
                    bad[w] += differ(x, y);
                }
            }
            uint64_t state = 0x9E3779B97F4A7C15ull * (w + 1);
            for (uint64_t i = 0; i < 250000000ull / stride; ++i) {
                state = state * 6364136223846793005ull + 1442695040888963407ull;
                const uint64_t r = state ^ (state >> 29);
                const uint32_t xb = static_cast<uint32_t>(r), yb = static_cast<uint32_t>(r >> 32);
                float x, y;
                memcpy(&x, &xb, 4);
                memcpy(&y, &yb, 4);
                if (i & 1) y = static_cast<float>(static_cast<int>(yb % 2001u) - 1000) / 64.0f;
                bad[w] += differ(x, y);
            }
        });
    }
    for (auto &t : pool) t.join();
    uint64_t sum = 0;
    for (uint64_t b : bad) sum += b;
    return sum;
}

// The f64 functions: `libm_check tanh|expm1 <stride>` draws 480 000 000 / stride inputs (arbitrary bits, (-25, 25),
// (-2, 2) and every binade down to 2^-70, a quarter each).
static uint64_t f64_differences(bool tanh_not_expm1, uint64_t stride) {
    const unsigned workers = std::max(1u, std::thread::hardware_concurrency());
    std::vector<uint64_t> bad(workers, 0);
    std::vector<std::thread> pool;
    for (unsigned w = 0; w < workers; ++w) {
        pool.emplace_back([&, w] {
            uint64_t state = 0xD1B54A32D192ED03ull * (w + 1);
            for (uint64_t i = 0; i < 480000000ull / stride / workers; ++i) {
                state = state * 6364136223846793005ull + 1442695040888963407ull;
                const uint64_t r = state ^ (state >> 31);
                const double unit = static_cast<double>(r >> 11) / 9007199254740992.0;
                double x;
                switch (i & 3) {
                    case 0: memcpy(&x, &r, 8); break;
                    case 1: x = (unit - 0.5) * 50.0; break;
                    case 2: x = (unit - 0.5) * 4.0; break;
                    default: x = std::ldexp(unit + 0.5, -static_cast<int>(r % 70)) * ((r & 1024) ? 1 : -1); break;
                }
                volatile double xv = x;
                const double want = tanh_not_expm1 ? tanh(xv) : expm1(xv);
                const double got = tanh_not_expm1 ? hmr::tanh_like_libm(x) : hmr::expm1_like_libm(x);
                uint64_t a, b;
                memcpy(&a, &want, 8);
                memcpy(&b, &got, 8);
                bad[w] += a != b && !(want != want && got != got);
            }
        });
    }
    for (auto &t : pool) t.join();
    uint64_t sum = 0;
    for (uint64_t b : bad) sum += b;
    return sum;
}

int main(int argc, char **argv) {
    if (argc >= 3 && (std::string(argv[1]) == "tanh" || std::string(argv[1]) == "expm1")) {
        std::printf("%llu differ\n", static_cast<unsigned long long>(f64_differences(std::string(argv[1]) == "tanh", strtoull(argv[2], nullptr, 10))));
        return 0;
    }
    if (argc >= 3 && std::string(argv[1]) == "powf") {
        const uint64_t stride = strtoull(argv[2], nullptr, 10);
        const bool fused = argc > 3 ? atoi(argv[3]) != 0 : true;
        std::printf("%llu differ\n", static_cast<unsigned long long>(fused ? powf_differences<true>(stride) : powf_differences<false>(stride)));
        return 0;
    }
    if (argc < 3) {
        std::fprintf(stderr, "usage: libm_check expf|expm1f|tanhf|log1pf|sinf|cosf|logf <stride> [fused]\n");
        return 2;
    }
    const std::string name = argv[1];
    const uint64_t stride = strtoull(argv[2], nullptr, 10);
    const bool fused = argc > 3 ? atoi(argv[3]) != 0 : true;
    const unsigned workers = std::max(1u, std::thread::hardware_concurrency());
    std::vector<uint64_t> bad(workers, 0);
    std::vector<uint32_t> first(workers, 0);
    std::vector<std::thread> pool;
    const uint64_t total = uint64_t{1} << 32, span = (total / workers / stride + 1) * stride;
    for (unsigned w = 0; w < workers; ++w) {
        pool.emplace_back([&, w] {
            const uint64_t begin = w * span, end = std::min(total, begin + span);
            auto run = [&](auto host, auto port) { bad[w] = count(begin, end, stride, &first[w], host, port); };
            if (name == "expf" && fused) run([](float x) { return expf(x); }, [](float x) { return hmr::expf_like_libm<true>(x); });
            else if (name == "expf") run([](float x) { return expf(x); }, [](float x) { return hmr::expf_like_libm<false>(x); });
            else if (name == "expm1f") run([](float x) { return expm1f(x); }, [](float x) { return hmr::expm1f_like_libm(x); });
            else if (name == "tanhf") run([](float x) { return tanhf(x); }, [](float x) { return hmr::tanhf_like_libm(x); });
            else if (name == "log1pf") run([](float x) { return log1pf(x); }, [](float x) { return hmr::log1pf_like_libm(x); });
            else if (name == "sinf" && fused) run([](float x) { return sinf(x); }, [](float x) { return hmr::sincosf_like_libm<true, false>(x); });
            else if (name == "sinf") run([](float x) { return sinf(x); }, [](float x) { return hmr::sincosf_like_libm<false, false>(x); });
            else if (name == "cosf" && fused) run([](float x) { return cosf(x); }, [](float x) { return hmr::sincosf_like_libm<true, true>(x); });
            else if (name == "cosf") run([](float x) { return cosf(x); }, [](float x) { return hmr::sincosf_like_libm<false, true>(x); });
            else if (name == "logf" && fused) run([](float x) { return logf(x); }, [](float x) { return hmr::logf_like_libm<true>(x); });
            else if (name == "logf") run([](float x) { return logf(x); }, [](float x) { return hmr::logf_like_libm<false>(x); });
            else bad[w] = ~uint64_t{0};
        });
    }
    for (auto &t : pool) t.join();
    uint64_t sum = 0;
    uint32_t example = 0;
    for (unsigned w = 0; w < workers; ++w) {
        if (bad[w] == ~uint64_t{0}) {
            std::fprintf(stderr, "unknown function %s\n", name.c_str());
            return 2;
        }
        if (bad[w] && !sum) example = first[w];
        sum += bad[w];
    }
    std::printf("%llu differ", static_cast<unsigned long long>(sum));
    if (sum) std::printf(" (first at bits 0x%08x)", example);
    std::printf("\n");
    return 0;
}
