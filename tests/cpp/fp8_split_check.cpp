// Host check of mfq_amd/csrc/fp8_split.h (the code the device runs): E4M3 rounding against the table of all 256 byte
// values (nearest, ties to even mantissa, saturation at 448), the block scale rule, and the accuracy of the hi + lo split.
#include "../../mfq_amd/csrc/fp8_split.h"

#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <random>
#include <vector>

using namespace mfq_amd::dev;

static void fail(const char* what, double a, double b) { std::fprintf(stderr, "%s: %.9g %.9g\n", what, a, b); std::exit(1); }

int main() {
    // the 127 finite non-negative values, ascending with the byte
    std::vector<float> table;
    for (int b = 0; b < 0x7f; ++b) {
        const float v = e4m3_to_float(static_cast<uint8_t>(b));
        const int e = (b >> 3) & 15, m = b & 7;
        const double expect = e == 0 ? m * std::ldexp(1.0, -9) : (1.0 + m / 8.0) * std::ldexp(1.0, e - 7);
        if (v != static_cast<float>(expect)) fail("e4m3_to_float", v, expect);
        if (!table.empty() && !(v > table.back())) fail("table order", v, table.back());
        table.push_back(v);
        if (e4m3_to_float(static_cast<uint8_t>(b | 0x80)) != -v) fail("sign", v, b);
    }
    if (table.back() != 448.0f) fail("largest", table.back(), 448);
    // rounding: brute force nearest with ties to the even byte, over a dense sweep and the exact midpoints
    std::mt19937_64 rng(5);
    std::uniform_real_distribution<double> exponent(-12.0, 9.5);
    long checked = 0;
    auto check = [&](float x) {
        const uint8_t got = e4m3_from_float(x);
        const float a = std::fabs(x);
        int best = 0;
        double best_distance = 1e30;
        for (int b = 0; b < 0x7f; ++b) {
            const double d = std::fabs(static_cast<double>(table[b]) - a);
            if (d < best_distance || (d == best_distance && (b & 1) == 0)) { best = b; best_distance = d; }
        }
        if (a >= 448.0f) best = 0x7e;
        const uint8_t expect = static_cast<uint8_t>(best | (std::signbit(x) ? 0x80 : 0));
        if (got != expect) fail("e4m3_from_float", x, got * 1000 + expect);
        ++checked;
    };
    for (int i = 0; i < 2000000; ++i) check(static_cast<float>((i & 1 ? -1.0 : 1.0) * std::exp2(exponent(rng))));
    for (size_t b = 0; b + 1 < table.size(); ++b) {
        const float mid = 0.5f * (table[b] + table[b + 1]);
        check(mid); check(-mid); check(std::nextafter(mid, 0.0f)); check(std::nextafter(mid, 1e9f));
        check(table[b]); check(-table[b]);
    }
    check(0.0f); check(-0.0f); check(448.0f); check(449.0f); check(1e30f); check(-1e30f); check(479.9f); check(1e-30f);
    // block scale: the smallest power of two that brings the block's largest magnitude to at most 448
    for (int i = 0; i < 200000; ++i) {
        const float largest = static_cast<float>(std::exp2(std::uniform_real_distribution<double>(-60.0, 60.0)(rng)));
        const uint8_t s = block_scale_byte(largest);
        const double scaled = static_cast<double>(largest) * std::ldexp(1.0, 127 - s);
        if (!(scaled <= 448.0 && scaled > 224.0)) fail("block_scale_byte", largest, scaled);
        if (scale_inverse(s) * scale_value(s) != 1.0f) fail("scale inverse", s, 0);
    }
    // the split: |x - (hi + lo)| <= 2^-8 |x| or one lo step, for every element of random blocks
    std::normal_distribution<float> normal(0.0f, 1.0f);
    double worst = 0.0;
    for (int trial = 0; trial < 20000; ++trial) {
        float x[32];
        const float spread = static_cast<float>(std::exp2(std::uniform_real_distribution<double>(-10.0, 10.0)(rng)));
        for (float& v : x) {
            v = normal(rng) * spread;
            uint32_t u = f32_bits(v) & 0xffff0000u;            // bf16-exact, as the kernels' inputs are
            v = bits_f32(u);
        }
        uint8_t hi[32], lo[32], s_hi, s_lo;
        split_block(x, hi, lo, s_hi, s_lo);
        double norm = 0.0, error = 0.0;
        for (int i = 0; i < 32; ++i) {
            const double back = static_cast<double>(e4m3_to_float(hi[i])) * std::ldexp(1.0, s_hi - 127) +
                                static_cast<double>(e4m3_to_float(lo[i])) * std::ldexp(1.0, s_lo - 127);
            norm += static_cast<double>(x[i]) * x[i];
            error += (back - x[i]) * (back - x[i]);
        }
        if (norm > 0.0) worst = std::fmax(worst, std::sqrt(error / norm));
    }
    if (!(worst < 4e-3)) fail("split accuracy", worst, 0);
    std::printf("%ld roundings checked; worst block rel-L2 of hi+lo %.3e\n", checked, worst);
    return 0;
}
