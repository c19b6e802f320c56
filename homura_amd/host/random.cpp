// Random sampling: the process-wide generator, the checks of every distribution and the reservation of Philox
// blocks, which is the same for every device (ref: src/ops/random.rs:14-360).
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <mutex>
#include <sstream>

#include "homura.hpp"

namespace homura {

namespace {

// ref: src/ops/random.rs:14-27
struct Generator {
    uint64_t seed = 67280421310721ull;  // PyTorch's default seed
    uint64_t offset = 0;                // Philox blocks handed out since seeding
};
std::mutex g_lock;
Generator g_generator;

// ref: src/ops/random.rs:65-72
void reserve_blocks(uint64_t blocks, uint64_t &seed, uint64_t &start) {
    std::lock_guard<std::mutex> lock(g_lock);
    seed = g_generator.seed;
    start = g_generator.offset;
    g_generator.offset += blocks;
}

int float_digits(DType dtype) { return dtype == DType::F16 ? 11 : dtype == DType::BF16 ? 8 : dtype == DType::F32 ? 24 : 53; }

// A number as Rust's `{}` prints an f64: the shortest digits that read back as the value, without an
// exponent (kept here for magnitudes beyond 10^21 or below 10^-7, where Rust writes every digit out).
std::string number(double v) {
    if (!std::isfinite(v)) return std::isnan(v) ? "NaN" : (v > 0 ? "inf" : "-inf");
    char buf[64];
    int precision = 0;
    for (precision = 0; precision < 17; ++precision) {
        std::snprintf(buf, sizeof buf, "%.*e", precision, v);
        if (std::strtod(buf, nullptr) == v) break;
    }
    const int exponent = v == 0.0 ? 0 : static_cast<int>(std::floor(std::log10(std::fabs(v))));
    if (exponent > 20 || exponent < -7) return buf;
    const int decimals = precision - exponent > 0 ? precision - exponent : 0;
    std::snprintf(buf, sizeof buf, "%.*f", decimals, v);
    return buf;
}

struct Dist {
    enum Kind { Uniform, Normal, Int } kind;
    double a = 0.0, b = 0.0;   // from, to / mean, std
    int64_t low = 0, high = 0;
};

// ref: src/ops/random.rs:113-177: runs before anything else, so a rejected call doesn't advance the generator.
void validate(const Dist &d, DType dtype) {
    if (d.kind != Dist::Int && !is_floating_point(dtype)) {
        throw Error(std::string("random floating point sampling is not implemented for ") + name_of(dtype) + " tensors");
    }
    if (d.kind == Dist::Uniform) {
        const double max = float_max(dtype);
        const std::pair<const char *, double> bounds[2] = {{"from", d.a}, {"to", d.b}};
        for (const auto &[name, v] : bounds) {
            if (!(v >= -max && v <= max)) {
                throw Error(std::string("uniform_ expects ") + name + " to be a finite value of " + name_of(dtype) + ", but got " +
                            name + "=" + number(v));
            }
        }
        if (d.a > d.b) {
            throw Error("uniform_ expects to return a [from, to) range, but found from=" + number(d.a) + " > to=" + number(d.b));
        }
        if (d.b - d.a > max) {
            throw Error("uniform_ expects to - from <= " + number(max) + " for " + name_of(dtype) + ", but got from=" + number(d.a) +
                        " and to=" + number(d.b));
        }
    } else if (d.kind == Dist::Normal) {
        if (std::isnan(d.b) || d.b < 0.0) throw Error("normal expects std >= 0.0, but found std " + number(d.b));
    } else {
        if (d.low >= d.high) {
            throw Error("random_ expects 'from' to be less than 'to', but got from=" + std::to_string(d.low) +
                        " >= to=" + std::to_string(d.high));
        }
        int64_t min, max;
        if (is_floating_point(dtype)) {
            max = int64_t{1} << float_digits(dtype);  // the integers every value of which the dtype represents
            min = -max;
        } else {
            int_range(dtype, min, max);
        }
        if (d.low < min || d.high - 1 > max) {
            throw Error("random_ expects [from, to) to lie inside [" + std::to_string(min) + ", " + std::to_string(max) + "] for " +
                        name_of(dtype) + ", but got from=" + std::to_string(d.low) + " and to=" + std::to_string(d.high));
        }
    }
}

uint64_t ceil_div(uint64_t a, uint64_t b) { return a / b + (a % b != 0); }

// ref: src/ops/random.rs:260-356
Tensor random_tensor(const Shape &shape, DType dtype, Device device, const Dist &d) {
    validate(d, dtype);
    for (int64_t s : shape) {
        if (s < 0) throw Error("a shape has no negative sizes");
    }
    if (d.kind != Dist::Int) {
        Tensor out = Tensor::uninit_on(shape, dtype, device);
        const uint64_t n = static_cast<uint64_t>(out.num_elements());
        uint64_t seed, start;
        if (d.kind == Dist::Uniform) {
            reserve_blocks(ceil_div(n, dtype == DType::F64 ? 2 : 4), seed, start);  // f64 takes two words per value
            backend::random_uniform(out.data(), seed, start, d.a, d.b);
        } else {
            reserve_blocks(ceil_div(n, 2), seed, start);  // Box-Muller: two normals per block
            backend::random_normal(out.data(), seed, start, d.a, d.b);
        }
        return out;
    }
    // Rejection sampling on 64-bit words, so that every value is equally likely: a word below 2^64 mod range is
    // dropped. Each batch reserves a block per two values still needed; the generator stays locked from the first
    // batch until the last one has advanced it (ref: src/ops/random.rs:217-258, 309-356).
    Tensor out = Tensor::uninit_on(shape, DType::I64, device);
    const uint64_t n = static_cast<uint64_t>(out.num_elements());
    const uint64_t range = static_cast<uint64_t>(d.high) - static_cast<uint64_t>(d.low);  // 1..=u64::MAX
    const uint64_t threshold = (0 - range) % range;
    std::optional<Tensor> workspace;
    if (threshold != 0 && device.kind == Device::K::Rocm) {
        const uint64_t tiles = ceil_div(ceil_div(n, 2), 256);
        workspace = Tensor::uninit_on(Shape{static_cast<int64_t>(2 * tiles + 1)}, DType::I64, device);
    }
    Tensor flat = out.reshape({static_cast<int64_t>(n)});
    {
        std::lock_guard<std::mutex> lock(g_lock);
        uint64_t done = 0;
        while (done < n) {
            const uint64_t needed = n - done, blocks = ceil_div(needed, 2), start = g_generator.offset;
            g_generator.offset += blocks;
            Tensor part = flat.narrow(0, static_cast<int64_t>(done), static_cast<int64_t>(needed));
            auto accepted = backend::random_int_batch(part.data(), g_generator.seed, start, blocks, d.low, range, threshold,
                                                      workspace ? &workspace->data() : nullptr);
            done += accepted ? std::min(*accepted, needed) : needed;
        }
    }
    return out.to(dtype);
}

}  // namespace

void manual_seed(uint64_t seed) {
    std::lock_guard<std::mutex> lock(g_lock);
    g_generator.seed = seed;
    g_generator.offset = 0;
}

Tensor rand(const Shape &shape, DType dtype, Device device) { return random_tensor(shape, dtype, device, Dist{Dist::Uniform, 0.0, 1.0}); }
Tensor randn(const Shape &shape, DType dtype, Device device) { return random_tensor(shape, dtype, device, Dist{Dist::Normal, 0.0, 1.0}); }
Tensor randint(int64_t low, int64_t high, const Shape &shape, DType dtype, Device device) {
    return random_tensor(shape, dtype, device, Dist{Dist::Int, 0.0, 0.0, low, high});
}
Tensor uniform(const Shape &shape, double from, double to, DType dtype, Device device) {
    return random_tensor(shape, dtype, device, Dist{Dist::Uniform, from, to});
}
Tensor normal(const Shape &shape, double mean, double std, DType dtype, Device device) {
    return random_tensor(shape, dtype, device, Dist{Dist::Normal, mean, std});
}

}  // namespace homura
