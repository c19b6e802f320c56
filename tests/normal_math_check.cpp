// Drives homura_amd/csrc/normal_math.hpp on the host: the same arithmetic as the GPU's Box-Muller pair,
// with hardware estimates that are cut down to 22 bits, against long double functions.
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <random>

#include "normal_math.hpp"

namespace {

double keep_22_bits(double x) {
    uint64_t b;
    memcpy(&b, &x, 8);
    b &= ~((uint64_t{1} << 30) - 1);
    memcpy(&x, &b, 8);
    return x;
}
struct CoarseSeeds {
    static double rcp(double x) { return keep_22_bits(1.0 / x); }
    static double rsq(double x) { return keep_22_bits(1.0 / std::sqrt(x)); }
};

double worst_log = 0, worst_root = 0, worst_turn = 0;
const long double kTwoPi = 6.283185307179586476925286766559L;

void relative(double got, long double want, double &worst, const char *what, double a, double b) {
    if (want == 0.0L) {
        if (got != 0.0) {
            std::printf("%s(%a, %a): %a where 0 is exact\n", what, a, b, got);
            std::exit(1);
        }
        return;
    }
    const double e = static_cast<double>(fabsl((static_cast<long double>(got) - want) / want));
    if (e > worst) worst = e;
}

void one(double u1, double u2) {
    const double l = hmr::normal_log<CoarseSeeds>(u1);
    relative(l, logl(static_cast<long double>(u1)), worst_log, "log", u1, 0);
    const double x = -2.0 * l;
    if (x == 0.0) {
        // Only u1 = 1 gets here; the root stands in for zero with a value no 32-bit output can hold.
        const double root = hmr::normal_sqrt<CoarseSeeds>(x);
        if (!(root >= 0.0 && root < 1.1e-150)) {
            std::printf("sqrt(0) gives %a\n", root);
            std::exit(1);
        }
    } else {
        relative(hmr::normal_sqrt<CoarseSeeds>(x), sqrtl(static_cast<long double>(x)), worst_root, "sqrt", x, 0);
    }
    double c, s;
    hmr::normal_turn(u2, c, s);
    // The reference reduces the same way (the difference is exact), so it is accurate next to a zero too.
    const int k = static_cast<int>(std::floor(4.0 * u2 + 0.5));
    const long double phi = kTwoPi * (static_cast<long double>(u2) - 0.25L * k);
    const long double cs[4] = {cosl(phi), -sinl(phi), -cosl(phi), sinl(phi)};
    const long double sn[4] = {sinl(phi), cosl(phi), -sinl(phi), -cosl(phi)};
    relative(c, cs[k & 3], worst_turn, "cos", u2, 0);
    relative(s, sn[k & 3], worst_turn, "sin", u2, 0);
}

}  // namespace

int main() {
    const double tiny = std::ldexp(1.0, -53);
    const double firsts[] = {tiny, 2 * tiny, 3 * tiny, 1e-10, 0.25, 0.5, 0.70710678118654746, 0.70710678118654757,
                             0.75, 1.0 - tiny, 1.0 - 2 * tiny, 1.0, 0.35355339059327379, 0.35355339059327373};
    double seconds[64];
    int m = 0;
    for (int q = 0; q <= 8; ++q) {
        const double at = q / 8.0;
        if (at < 1.0) seconds[m++] = at;
        if (at > 0.0) seconds[m++] = at - tiny, seconds[m++] = at - 3 * tiny;
        if (at < 1.0) seconds[m++] = at + tiny, seconds[m++] = at + 5 * tiny;
    }
    for (double u1 : firsts)
        for (int j = 0; j < m; ++j) one(u1, seconds[j]);
    std::mt19937_64 gen(7);
    for (int i = 0; i < 3000000; ++i) {
        const double a = static_cast<double>(gen() >> 11) * tiny, b = static_cast<double>(gen() >> 11) * tiny;
        one(1.0 - a, b);
        // Small first arguments and second arguments close to the quarter turns are rare in a uniform draw.
        if (i % 8 == 0) one(std::ldexp(1.0 - a * 0.5, -static_cast<int>(gen() % 53)), std::floor(b * 8.0) / 8.0 + b * 1e-9);
    }
    std::printf("log %.3g sqrt %.3g turn %.3g\n", worst_log, worst_root, worst_turn);
    const double limit = std::ldexp(1.0, -49);
    if (worst_log > limit || worst_root > limit || worst_turn > limit) {
        std::printf("over 2^-49\n");
        return 1;
    }
    std::printf("normal math ok\n");
    return 0;
}
