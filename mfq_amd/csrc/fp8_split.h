// Activations as two OCP FP8 (E4M3) operands with E8M0 block scales, for the block-scaled MFMA of gfx950:
//   x  ~=  hi * 2^(s_hi - 127)  +  lo * 2^(s_lo - 127)      per block of 32 consecutive columns
// hi carries the value rounded to E4M3 at the block's scale, lo the residual (exact in fp32 for fp16 / bf16 inputs)
// rounded to E4M3 at a scale of its own.  Plain integer / float code that compiles for the device and for the host
// (tests/cpp/fp8_split_check.cpp checks the rounding against every E4M3 value).
#pragma once

#include <stdint.h>
#include <string.h>

#if defined(__HIPCC__)
#define MFQ_HD __host__ __device__ __forceinline__
#else
#define MFQ_HD inline
#endif

namespace mfq_amd {
namespace dev {

MFQ_HD uint32_t f32_bits(float v) { uint32_t u; memcpy(&u, &v, 4); return u; }
MFQ_HD float bits_f32(uint32_t u) { float v; memcpy(&v, &u, 4); return v; }

// Value of an E4M3 byte (OCP "FN": no infinities, 0x7f / 0xff are NaN, largest finite 448).
MFQ_HD float e4m3_to_float(uint8_t b) {
    const uint32_t sign = static_cast<uint32_t>(b & 0x80u) << 24;
    const uint32_t exponent = (b >> 3) & 15u, mantissa = b & 7u;
    float magnitude;
    if (exponent == 0) magnitude = static_cast<float>(mantissa) * 0.001953125f;            // subnormal: m * 2^-9
    else magnitude = bits_f32(((exponent + 120u) << 23) | (mantissa << 20));                // (1 + m/8) * 2^(e-7)
    return bits_f32(f32_bits(magnitude) | sign);
}

// Round to nearest even, saturating at +-448; NaN becomes 0 (the inputs here are finite).
MFQ_HD uint8_t e4m3_from_float(float v) {
    const uint32_t u = f32_bits(v);
    const uint8_t sign = static_cast<uint8_t>((u >> 24) & 0x80u);
    const float a = bits_f32(u & 0x7fffffffu);
    if (!(a == a)) return 0;
    if (a >= 448.0f) return static_cast<uint8_t>(sign | 0x7eu);
    if (a < 0.015625f) {
        // below the smallest normal (2^-6): multiples of 2^-9; adding 2^14 * 2^-9... rounds to nearest even in fp32
        const float scaled = a * 512.0f;                                  // exact
        const float rounded = (scaled + 8388608.0f) - 8388608.0f;         // RNE to an integer 0..8
        return static_cast<uint8_t>(sign | static_cast<uint8_t>(rounded)); // 8 is the smallest normal, 0x08
    }
    // normal: keep 3 mantissa bits, round to nearest even on the 20 dropped bits
    const uint32_t bits = f32_bits(a);
    const uint32_t rounded = bits + 0x7ffffu + ((bits >> 20) & 1u);
    const uint32_t exponent = (rounded >> 23) - 120u, mantissa = (rounded >> 20) & 7u;    // exponent 1..15
    const uint32_t byte = (exponent << 3) | mantissa;
    return static_cast<uint8_t>(sign | (byte > 0x7eu ? 0x7eu : byte));
}

// E8M0 byte s of the smallest power of two 2^(s-127) with largest / 2^(s-127) <= 448 (s >= 1; 127 for a zero block).
MFQ_HD uint8_t block_scale_byte(float largest) {
    if (!(largest > 0.0f)) return 127;
    const uint32_t u = f32_bits(largest);
    int exponent = static_cast<int>((u >> 23) & 0xffu) - 127;             // largest = m * 2^exponent, 1 <= m < 2 (subnormals: rare, see below)
    const uint32_t mantissa = u & 0x7fffffu;
    if (((u >> 23) & 0xffu) == 0) exponent = -126;
    int e = exponent - 8 + (mantissa > 0x600000u ? 1 : 0);                // 448 = 1.75 * 2^8
    e = e < -126 ? -126 : e > 127 ? 127 : e;
    return static_cast<uint8_t>(e + 127);
}
MFQ_HD float scale_inverse(uint8_t s) { return bits_f32(static_cast<uint32_t>(254 - s) << 23); }   // 2^-(s-127), s in 1..253
MFQ_HD float scale_value(uint8_t s) { return bits_f32(static_cast<uint32_t>(s) << 23); }            // 2^(s-127), s in 1..254

// One block of 32 values: hi[32], lo[32] and their two scale bytes.
MFQ_HD void split_block(const float (&x)[32], uint8_t (&hi)[32], uint8_t (&lo)[32], uint8_t& s_hi, uint8_t& s_lo) {
    float largest = 0.0f;
    for (int i = 0; i < 32; ++i) { const float a = x[i] < 0.0f ? -x[i] : x[i]; largest = a > largest ? a : largest; }
    s_hi = block_scale_byte(largest);
    const float down = scale_inverse(s_hi), up = scale_value(s_hi);
    float residual[32], largest_residual = 0.0f;
    for (int i = 0; i < 32; ++i) {
        hi[i] = e4m3_from_float(x[i] * down);
        residual[i] = x[i] - e4m3_to_float(hi[i]) * up;
        const float a = residual[i] < 0.0f ? -residual[i] : residual[i];
        largest_residual = a > largest_residual ? a : largest_residual;
    }
    s_lo = block_scale_byte(largest_residual);
    const float down_lo = scale_inverse(s_lo);
    for (int i = 0; i < 32; ++i) lo[i] = e4m3_from_float(residual[i] * down_lo);
}

}  // namespace dev
}  // namespace mfq_amd
